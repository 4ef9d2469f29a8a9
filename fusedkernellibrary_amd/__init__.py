"""Python host side of the MI355X-native fused Transform path.

The product is the C++17 template library under include/fk/ (the operator API: PerThreadRead, .then(), Crop, Resize,
Mul/Sub/Div, ColorConversion, TensorWrite, executeOperations) and its hand-written gfx950 kernels.  This module only
loads the two native libraries built from it and exposes the chain entry points of include/fk_capi.h to Python, with
torch tensors as device memory.  There is no CPU or eager fallback: if the native library is missing, or a call fails,
an exception is raised.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))

PRESERVE_AR, IGNORE_AR, PRESERVE_AR_RN_EVEN, PRESERVE_AR_LEFT = 0, 1, 2, 3
# (batches take any number of planes: it is a run-time value at the C boundary)
CHAIN_DEPTHS = (1, 2, 4, 8, 16, 32, 64, 128)


class FkError(RuntimeError):
    pass


class Rect(C.Structure):
    _fields_ = [("x", C.c_int), ("y", C.c_int), ("width", C.c_int), ("height", C.c_int)]


def _rects(rects):
    arr = (Rect * len(rects))()
    for i, r in enumerate(rects):
        arr[i] = Rect(*[int(v) for v in r])
    return arr


def _f3(v):
    return (C.c_float * 3)(*[float(x) for x in v])


_vp, _i, _f, _sz = C.c_void_p, C.c_int, C.c_float, C.c_size_t
_f3p = C.POINTER(C.c_float)
_rp = C.POINTER(Rect)

CAPI_SIGNATURES = {
    "fk_crop_resize_muls_bgr_tensor": [_vp, _i, _i, _sz, _rp, _i, _i, _i, _i, _f3p, _f3p, _f3p, _f3p, _vp, _vp],
    "fk_crop_resize_muls_bgr_tensor_noalloc": [_vp, _i, _i, _sz, _rp, _i, _i, _i, _i, _f3p, _f3p, _f3p, _f3p, _vp, _vp],
    "fk_muladd_chain_f32c3": [_vp, _i, _i, _sz, _i, _f, _f, _vp, _sz, _vp],
    "fk_single_op_f32c3": [_vp, _i, _i, _sz, _i, _f, _vp, _sz, _vp],
    "fk_batch_crop_resize_norm_split": [C.POINTER(C.c_void_p), _i, _i, _sz, _rp, _i, _i, _i, _f3p, _f3p, _f3p, _vp, _vp],
    "fk_resize_crop_tiles": [_vp, _i, _i, _sz, _i, _i, _rp, _i, _i, _i, _f3p, _vp, _vp],
    "fk_rgba2gray_u8c4": [_vp, _i, _i, _sz, _vp, _sz, _vp],
    "fk_resize_mul_u8c4_f32c4": [_vp, _i, _i, _sz, _i, _i, _f, _vp, _sz, _vp],
    "fk_crop_mul_saturate_u8c4": [_vp, _i, _i, _sz, Rect, _i, _vp, _sz, _vp],
    "fk_rgba2bgr_sub_u8c4_f32c3": [_vp, _i, _i, _sz, _f, _vp, _sz, _vp],
    "fk_divergent4_u8c4": [_vp, _i, _i, _sz, _vp, _i, _i, _f, _vp, Rect, _i, _vp, _f, _vp, _vp],
    "fk_batch_crop_cast_tensor": [_vp, _i, _i, _sz, _rp, _i, _i, _i, _vp, _vp],
    "fk_batch_windows_saturate_muls_f32": [_vp, _i, _i, _sz, _rp, _i, _f, _f, _f, _vp, _vp],
    "fk_read_yuv": [_i, _vp, _sz, _i, _i, _vp, _sz, _vp],
    "fk_write_yuv": [_i, _vp, _sz, _i, _i, _vp, _sz, _vp],
    "fk_yuv_to_rgb": [_i, _i, _i, _i, _i, _vp, _sz, _i, _i, _vp, _sz, _vp],
    "fk_yuv_crop_resize_norm_split": [_i, _i, _i, _vp, _sz, _i, _i, Rect, _i, _i, _f, _vp, _vp],
    "fk_border_crop_u8c3": [_i, _vp, _i, _i, _sz, _i, _i, _i, _i, C.POINTER(C.c_uint8), _vp, _sz, _vp],
    "fk_warp_u8c3_f32c3": [_i, C.POINTER(C.c_float), _vp, _i, _i, _sz, _i, _i, _vp, _sz, _vp],
    "fk_deinterlace_u8c3_f32c3": [_i, _i, _vp, _i, _i, _sz, _vp, _sz, _vp],
    "fk_tensor_relayout_f32c3": [_i, _vp, _i, _i, _i, _vp, _vp],
    "fk_circular_tensor_read_f32c3": [_i, _i, _vp, _i, _i, _i, _vp, _vp],
    "fk_circular_tensor_update_u8c3_split_f32": [_vp, _i, _i, _sz, _f, _vp, _vp, _i, _i, _i, _vp],
    "fk_conditional_copy_u8c3": [C.POINTER(C.c_void_p), _i, _i, _sz, _i, _i, C.POINTER(C.c_uint8), _vp, _vp],
    "fk_conditional_resize_f32c3": [C.POINTER(C.c_void_p), _i, _i, _sz, _i, _i, _f3p, _i, _i, _vp, _vp],
    "fk_muladd_midwrite_f32c3": [_vp, _i, _i, _sz, _f, _f, _vp, _sz, _vp, _sz, _vp],
    "fk_batch_crop_cast_images": [_vp, _i, _i, _sz, _rp, _i, C.POINTER(C.c_void_p), _sz, _vp],
    "fk_tensor_mul_f32c3": [_vp, _i, _i, _i, _f3p, _vp, _vp],
    "fk_set_to_f32c3_tensor": [_f3p, _vp, _i, _i, _i, _vp],
}
PACKED_TO_SPLIT, PACKED_TO_TRANSPOSED, SPLIT_TO_PACKED, TRANSPOSED_TO_PACKED = 0, 1, 2, 3
ASCENDENT, DESCENDENT = 0, 1
BORDER_CONSTANT, BORDER_REPLICATE, BORDER_REFLECT, BORDER_WRAP, BORDER_REFLECT_101 = 0, 1, 2, 3, 4
WARP_AFFINE, WARP_PERSPECTIVE = 0, 1
DEINTERLACE_BLEND, DEINTERLACE_INTER_LINEAR = 0, 1
# PixelFormat / ColorRange / ColorPrimitives values of include/fk_capi.h
NV12, NV21, P010, P210, Y210, UYVY = 0, 1, 3, 6, 8, 10
RANGE_LIMITED, RANGE_FULL = 0, 1
BT601, BT709, BT2020 = 0, 1, 2
RUNTIME_SYMBOLS = [
    "fkrt_device_count", "fkrt_set_device", "fkrt_get_device", "fkrt_stream_create", "fkrt_stream_destroy",
    "fkrt_stream_sync", "fkrt_malloc", "fkrt_malloc_pitch", "fkrt_free", "fkrt_malloc_host", "fkrt_free_host",
    "fkrt_memcpy_async", "fkrt_memcpy2d_async", "fkrt_memset_async", "fkrt_launch", "fkrt_params_upload",
    "fkrt_params_release", "fkrt_max_kernarg_bytes", "fkrt_last_error", "fkrt_error_string", "fkrt_event_create", "fkrt_event_destroy",
    "fkrt_event_record", "fkrt_event_sync", "fkrt_event_elapsed_ms",
]

_libs = {}


def library_paths():
    return os.path.join(_HERE, "libfk_hip_rt.so"), os.path.join(_HERE, "libfk_capi.so")


def use_literal_interpolation(enable=True):
    """Switch the chain entry points to libfk_capi_literal.so, built with the reference's host-branch bilinear
    interpolation (row index from the x coordinate).  For parity demonstrations against the reference CPU backend."""
    _libs.pop("capi", None)
    _libs["variant"] = "libfk_capi_literal.so" if enable else "libfk_capi.so"


def load():
    """Load (once) and return (runtime, capi) ctypes handles; raises FkError when they have not been built."""
    if "capi" not in _libs:
        rt_path, capi_path = library_paths()
        capi_path = os.path.join(_HERE, _libs.get("variant", "libfk_capi.so"))
        for p in (rt_path, capi_path):
            if not os.path.exists(p):
                raise FkError(f"native library {p} is missing: build it with `python -m fusedkernellibrary_amd.build`")
        rt = C.CDLL(rt_path, mode=C.RTLD_GLOBAL)
        capi = C.CDLL(capi_path)
        for name, sig in CAPI_SIGNATURES.items():
            fn = getattr(capi, name)
            fn.argtypes = sig
            fn.restype = C.c_int
        capi.fk_last_error.restype = C.c_char_p
        capi.fk_interpolate_y1_from_x.restype = C.c_int
        rt.fkrt_error_string.restype = C.c_char_p
        rt.fkrt_error_string.argtypes = [C.c_int]
        rt.fkrt_max_kernarg_bytes.restype = C.c_size_t
        rt.fkrt_event_create.argtypes = [C.POINTER(C.c_void_p)]
        rt.fkrt_event_destroy.argtypes = [C.c_void_p]
        rt.fkrt_event_record.argtypes = [C.c_void_p, C.c_void_p]
        rt.fkrt_event_sync.argtypes = [C.c_void_p]
        rt.fkrt_event_elapsed_ms.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        rt.fkrt_stream_create.argtypes = [C.POINTER(C.c_void_p)]
        rt.fkrt_stream_destroy.argtypes = [C.c_void_p]
        rt.fkrt_stream_sync.argtypes = [C.c_void_p]
        _libs["rt"], _libs["capi"] = rt, capi
    return _libs["rt"], _libs["capi"]


def _check(rc):
    if rc != 0:
        _, capi = load()
        kinds = {1: "unsupported", 2: "runtime", 3: "argument"}
        raise FkError(f"fk call failed ({kinds.get(rc, rc)}): {capi.fk_last_error().decode()}")


def _call(fn, args, defer):
    """Run the entry point now, or (defer=True) return a zero-argument callable that runs it with these already
    marshalled arguments: for tight launch loops that should not pay the marshalling again."""
    if defer:
        def run():
            rc = fn(*args)
            if rc != 0:
                _check(rc)
        return run
    _check(fn(*args))
    return None


def _stream(stream):
    if stream is not None:
        return C.c_void_p(stream)
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(t, dtype_name):
    import torch
    if not t.is_cuda:
        raise FkError("tensors must live on the GPU")
    if t.dtype != getattr(torch, dtype_name):
        raise FkError(f"expected a {dtype_name} tensor")
    if t.stride(-1) != 1 or (t.dim() >= 3 and t.stride(-2) != t.shape[-1]):
        raise FkError("pixels must be contiguous along a row")
    return t


def _image(t, dtype_name):
    """(h, w, c) tensor whose row stride is the pitch -> (ptr, w, h, pitch_bytes)."""
    t = _dev(t, dtype_name)
    h, w = t.shape[0], t.shape[1]
    return C.c_void_p(t.data_ptr()), w, h, t.stride(0) * t.element_size()


# ---- chains: each mirrors one entry point of include/fk_capi.h; outputs are written into `out` ----------------------

def crop_resize_muls_bgr_tensor(src, rects, out, aspect, background, mul, sub, div, stream=None, defer=False):
    """README pipeline. src: (H, W, 3) uint8; out: (n, dst_h, dst_w, 3) float32 contiguous."""
    _, capi = load()
    p, w, h, pitch = _image(src, "uint8")
    out = _dev(out, "float32")
    n, dh, dw, _ = out.shape
    assert n == len(rects) and out.is_contiguous()
    _deferred = _call(capi.fk_crop_resize_muls_bgr_tensor, (p, w, h, pitch, _rects(rects), n, dw, dh, aspect, _f3(background), _f3(mul),
                                               _f3(sub), _f3(div), C.c_void_p(out.data_ptr()), _stream(stream)), defer)
    return _deferred if defer else out


def crop_resize_muls_bgr_tensor_noalloc(src, rects, out, aspect, background, mul, sub, div, stream=None, defer=False):
    """The README pipeline through the entry point that allocates nothing (at most 64 planes); same arguments and results."""
    _, capi = load()
    p, w, h, pitch = _image(src, "uint8")
    out = _dev(out, "float32")
    n, dh, dw, _ = out.shape
    assert n == len(rects) and out.is_contiguous()
    _deferred = _call(capi.fk_crop_resize_muls_bgr_tensor_noalloc, (p, w, h, pitch, _rects(rects), n, dw, dh, aspect, _f3(background), _f3(mul),
                                                                      _f3(sub), _f3(div), C.c_void_p(out.data_ptr()), _stream(stream)), defer)
    return _deferred if defer else out


def muladd_chain_f32c3(src, dst, depth, mul_v, add_v, stream=None, defer=False):
    _, capi = load()
    p, w, h, pitch = _image(src, "float32")
    q, w2, h2, pitch2 = _image(dst, "float32")
    assert (w, h) == (w2, h2)
    _deferred = _call(capi.fk_muladd_chain_f32c3, (p, w, h, pitch, depth, mul_v, add_v, q, pitch2, _stream(stream)), defer)
    return _deferred if defer else dst


def single_op_f32c3(src, dst, is_add, v, stream=None, defer=False):
    _, capi = load()
    p, w, h, pitch = _image(src, "float32")
    q, w2, h2, pitch2 = _image(dst, "float32")
    assert (w, h) == (w2, h2)
    _deferred = _call(capi.fk_single_op_f32c3, (p, w, h, pitch, int(is_add), v, q, pitch2, _stream(stream)), defer)
    return _deferred if defer else dst


def batch_crop_resize_norm_split(srcs, rects, out, div1, sub, div2, stream=None, defer=False):
    """srcs: list of (H, W, 3) uint8 of one size/pitch; out: (n, 3, dst_h, dst_w) float32 contiguous."""
    _, capi = load()
    n = len(srcs)
    p0, w, h, pitch = _image(srcs[0], "uint8")
    for s in srcs:
        assert _image(s, "uint8")[1:] == (w, h, pitch)
    ptrs = (C.c_void_p * n)(*[s.data_ptr() for s in srcs])
    out = _dev(out, "float32")
    assert out.shape[0] == n == len(rects) and out.shape[1] == 3 and out.is_contiguous()
    _deferred = _call(capi.fk_batch_crop_resize_norm_split, (ptrs, w, h, pitch, _rects(rects), n, out.shape[3], out.shape[2], _f3(div1),
                                                _f3(sub), _f3(div2), C.c_void_p(out.data_ptr()), _stream(stream)), defer)
    return _deferred if defer else out


def resize_crop_tiles(src, resized, rects, out, mul, stream=None, defer=False):
    """src: (H, W, 3) uint8; resized = (rs_w, rs_h); out: (n, tile_h, tile_w, 3) float32 contiguous."""
    _, capi = load()
    p, w, h, pitch = _image(src, "uint8")
    out = _dev(out, "float32")
    n, th, tw, _ = out.shape
    assert n == len(rects) and out.is_contiguous()
    _deferred = _call(capi.fk_resize_crop_tiles, (p, w, h, pitch, resized[0], resized[1], _rects(rects), n, tw, th, _f3(mul),
                                     C.c_void_p(out.data_ptr()), _stream(stream)), defer)
    return _deferred if defer else out


def rgba2gray_u8c4(src, dst, stream=None, defer=False):
    _, capi = load()
    p, w, h, pitch = _image(src, "uint8")
    d = _dev(dst, "uint8")
    _deferred = _call(capi.fk_rgba2gray_u8c4, (p, w, h, pitch, C.c_void_p(d.data_ptr()), d.stride(0), _stream(stream)), defer)
    return _deferred if defer else dst


def resize_mul_u8c4_f32c4(src, dst, mul_v, stream=None, defer=False):
    _, capi = load()
    p, w, h, pitch = _image(src, "uint8")
    q, dw, dh, dpitch = _image(dst, "float32")
    _deferred = _call(capi.fk_resize_mul_u8c4_f32c4, (p, w, h, pitch, dw, dh, mul_v, q, dpitch, _stream(stream)), defer)
    return _deferred if defer else dst


def crop_mul_saturate_u8c4(src, rect, dst, mul_v, stream=None, defer=False):
    _, capi = load()
    p, w, h, pitch = _image(src, "uint8")
    q, _, _, dpitch = _image(dst, "uint8")
    _deferred = _call(capi.fk_crop_mul_saturate_u8c4, (p, w, h, pitch, Rect(*rect), mul_v, q, dpitch, _stream(stream)), defer)
    return _deferred if defer else dst


def rgba2bgr_sub_u8c4_f32c3(src, dst, sub_v, stream=None, defer=False):
    _, capi = load()
    p, w, h, pitch = _image(src, "uint8")
    q, _, _, dpitch = _image(dst, "float32")
    _deferred = _call(capi.fk_rgba2bgr_sub_u8c4_f32c3, (p, w, h, pitch, sub_v, q, dpitch, _stream(stream)), defer)
    return _deferred if defer else dst


def divergent4_u8c4(src, gray_out, resized_out, mul_b, rect_c, mul_c, crop_out, sub_d, bgr_out, stream=None, defer=False):
    """All four chains in one launch; outputs must be contiguous."""
    _, capi = load()
    p, w, h, pitch = _image(src, "uint8")
    for t in (gray_out, resized_out, crop_out, bgr_out):
        assert t.is_contiguous()
    _deferred = _call(capi.fk_divergent4_u8c4, (p, w, h, pitch, C.c_void_p(_dev(gray_out, "uint8").data_ptr()), resized_out.shape[1],
                                   resized_out.shape[0], mul_b, C.c_void_p(_dev(resized_out, "float32").data_ptr()),
                                   Rect(*rect_c), mul_c, C.c_void_p(_dev(crop_out, "uint8").data_ptr()), sub_d,
                                   C.c_void_p(_dev(bgr_out, "float32").data_ptr()), _stream(stream)), defer)
    return _deferred


def batch_crop_cast_tensor(src, rects, out, stream=None, defer=False):
    """out: (n, max_h, max_w, 3) float32 contiguous; elements outside a plane's own rect stay untouched."""
    _, capi = load()
    p, w, h, pitch = _image(src, "uint8")
    out = _dev(out, "float32")
    n, mh, mw, _ = out.shape
    assert n == len(rects) and out.is_contiguous()
    _deferred = _call(capi.fk_batch_crop_cast_tensor, (p, w, h, pitch, _rects(rects), n, mw, mh, C.c_void_p(out.data_ptr()), _stream(stream)), defer)
    return _deferred if defer else out


def batch_windows_saturate_muls_f32(src, rects, out, mul_v, sub_v, div_v, stream=None, defer=False):
    """The reference's horizontal-fusion benchmark chain. src: (H, W) uint8 whose row stride is the pitch; rects of one size;
    out: (n, rect_h, rect_w) float32 contiguous."""
    _, capi = load()
    t = _dev(src, "uint8")
    if t.dim() != 2:
        raise FkError("expected a (h, w) image of bytes")
    out = _dev(out, "float32")
    assert out.shape == (len(rects), rects[0][3], rects[0][2]) and out.is_contiguous()
    _deferred = _call(capi.fk_batch_windows_saturate_muls_f32, (C.c_void_p(t.data_ptr()), t.shape[1], t.shape[0], t.stride(0), _rects(rects), len(rects),
                                                                float(mul_v), float(sub_v), float(div_v), C.c_void_p(out.data_ptr()), _stream(stream)), defer)
    return _deferred if defer else out


# ---- YUV front-end: `raw` is the 2D buffer of base elements (uint8, or uint16/int16 for 10-bit formats) ------------

def _raw(t, fmt):
    import torch
    if not t.is_cuda or t.dim() != 2 or t.stride(1) != 1:
        raise FkError("a raw YUV image is a 2D GPU tensor with contiguous rows")
    wide = fmt in (P010, P210, Y210)
    if t.dtype not in ((torch.uint16, torch.int16) if wide else (torch.uint8,)):
        raise FkError("raw YUV image has the wrong element type for its format")
    return C.c_void_p(t.data_ptr()), t.stride(0) * t.element_size()


def _pixels(t):
    if not t.is_cuda or t.dim() != 3 or t.stride(2) != 1 or t.stride(1) != t.shape[2]:
        raise FkError("pixels must be a (h, w, c) GPU tensor, contiguous along a row")
    return C.c_void_p(t.data_ptr()), t.stride(0) * t.element_size()


def read_yuv(fmt, raw, out, stream=None, defer=False):
    """raw image -> out: (h, w, 3) {Y, U, V} pixels of the raw element type."""
    _, capi = load()
    p, pitch = _raw(raw, fmt)
    q, out_pitch = _pixels(out)
    h, w, _ = out.shape
    _deferred = _call(capi.fk_read_yuv, (fmt, p, pitch, w, h, q, out_pitch, _stream(stream)), defer)
    return _deferred if defer else out


def write_yuv(fmt, pixels, raw, stream=None, defer=False):
    """(h, w, 3) {Y, U, V} pixels -> raw image."""
    _, capi = load()
    p, pitch = _pixels(pixels)
    q, raw_pitch = _raw(raw, fmt)
    h, w, _ = pixels.shape
    _deferred = _call(capi.fk_write_yuv, (fmt, p, pitch, w, h, q, raw_pitch, _stream(stream)), defer)
    return _deferred if defer else raw


def yuv_to_rgb(fmt, color_range, primaries, raw, out, stream=None, defer=False):
    """raw image -> out: (h, w, 3 or 4) RGB[A] pixels, of the raw element type or float32."""
    import torch
    _, capi = load()
    p, pitch = _raw(raw, fmt)
    q, out_pitch = _pixels(out)
    h, w, cn = out.shape
    if cn not in (3, 4):
        raise FkError("output pixels have 3 or 4 channels")
    _deferred = _call(capi.fk_yuv_to_rgb, (fmt, color_range, primaries, int(cn == 4), int(out.dtype == torch.float32), p, pitch, w, h, q,
                                           out_pitch, _stream(stream)), defer)
    return _deferred if defer else out


def yuv_crop_resize_norm_split(fmt, color_range, primaries, raw, size, crop, out, div_v, stream=None, defer=False):
    """raw image of size = (w, h) -> RGB -> crop (x, y, w, h) -> resize -> / div_v -> out: (3, dst_h, dst_w) float32."""
    _, capi = load()
    p, pitch = _raw(raw, fmt)
    out = _dev(out, "float32")
    _, dh, dw = out.shape
    assert out.is_contiguous()
    _deferred = _call(capi.fk_yuv_crop_resize_norm_split, (fmt, color_range, primaries, p, pitch, size[0], size[1], Rect(*[int(v) for v in crop]),
                                                           dw, dh, float(div_v), C.c_void_p(out.data_ptr()), _stream(stream)), defer)
    return _deferred if defer else out


# ---- BorderReader and Warping ------------------------------------------------------------------------------------------

def border_crop_u8c3(border_type, src, left, top, out, value=(0, 0, 0), stream=None, defer=False):
    """src: (h, w, 3) uint8 seen through BorderReader<border_type>; out: (dst_h, dst_w, 3) uint8 = the window whose origin
    is (-left, -top) in image coordinates."""
    _, capi = load()
    p, w, h, pitch = _image(src, "uint8")
    q, dw, dh, out_pitch = _image(out, "uint8")
    val = (C.c_uint8 * 3)(*[int(v) for v in value])
    _deferred = _call(capi.fk_border_crop_u8c3, (border_type, p, w, h, pitch, int(left), int(top), dw, dh, val, q, out_pitch, _stream(stream)), defer)
    return _deferred if defer else out


def warp_u8c3_f32c3(warp_type, matrix, src, out, stream=None, defer=False):
    """matrix: 6 (affine) or 9 (perspective) floats, row-major, destination -> source; out: (dst_h, dst_w, 3) float32."""
    _, capi = load()
    p, w, h, pitch = _image(src, "uint8")
    q, dw, dh, out_pitch = _image(out, "float32")
    flat = [float(v) for row in matrix for v in (row if hasattr(row, "__len__") else [row])]
    if len(flat) != (6 if warp_type == WARP_AFFINE else 9):
        raise FkError("matrix must be 2x3 (affine) or 3x3 (perspective)")
    m = (C.c_float * len(flat))(*flat)
    _deferred = _call(capi.fk_warp_u8c3_f32c3, (warp_type, m, p, w, h, pitch, dw, dh, q, out_pitch, _stream(stream)), defer)
    return _deferred if defer else out


def deinterlace_u8c3_f32c3(kind, use_even_lines, src, out, stream=None, defer=False):
    """src: (h, w, 3) uint8; out: (h, w, 3) float32."""
    _, capi = load()
    p, w, h, pitch = _image(src, "uint8")
    q, ow, oh, out_pitch = _image(out, "float32")
    assert (ow, oh) == (w, h)
    _deferred = _call(capi.fk_deinterlace_u8c3_f32c3, (kind, int(use_even_lines), p, w, h, pitch, q, out_pitch, _stream(stream)), defer)
    return _deferred if defer else out


# ---- tensor layouts and circular tensors ------------------------------------------------------------------------------

def tensor_relayout_f32c3(mode, src, w, h, planes, out, stream=None, defer=False):
    """src / out: contiguous float32 tensors of planes*h*w*3 elements in the layouts the mode names."""
    _, capi = load()
    src, out = _dev(src, "float32"), _dev(out, "float32")
    assert src.is_contiguous() and out.is_contiguous() and src.numel() == out.numel() == planes * h * w * 3
    _deferred = _call(capi.fk_tensor_relayout_f32c3, (mode, C.c_void_p(src.data_ptr()), w, h, planes, C.c_void_p(out.data_ptr()), _stream(stream)), defer)
    return _deferred if defer else out


def circular_tensor_read_f32c3(direction, first, ring, out, stream=None, defer=False):
    """ring / out: (planes, h, w, 3) float32 contiguous."""
    _, capi = load()
    ring, out = _dev(ring, "float32"), _dev(out, "float32")
    planes, h, w, _ = ring.shape
    assert ring.is_contiguous() and out.is_contiguous() and out.shape == ring.shape
    _deferred = _call(capi.fk_circular_tensor_read_f32c3, (direction, first, C.c_void_p(ring.data_ptr()), w, h, planes, C.c_void_p(out.data_ptr()),
                                                          _stream(stream)), defer)
    return _deferred if defer else out


def circular_tensor_update_u8c3_split_f32(frame, mul_v, tensor, ring, next_index, newest_first, stream=None, defer=False):
    """frame: (h, w, 3) uint8; tensor, ring: (batch, 3, h, w) float32 contiguous, updated in place.  Returns the ring
    slot for the next update."""
    _, capi = load()
    p, w, h, pitch = _image(frame, "uint8")
    tensor, ring = _dev(tensor, "float32"), _dev(ring, "float32")
    batch = tensor.shape[0]
    assert tensor.is_contiguous() and ring.is_contiguous() and tuple(tensor.shape) == tuple(ring.shape) == (batch, 3, h, w)
    _deferred = _call(capi.fk_circular_tensor_update_u8c3_split_f32, (p, w, h, pitch, float(mul_v), C.c_void_p(tensor.data_ptr()), C.c_void_p(ring.data_ptr()),
                                                                     batch, next_index, int(newest_first), _stream(stream)), defer)
    return _deferred if defer else (next_index + 1) % batch


# ---- less common chain shapes: conditional batches, a write in the middle of a chain, a batch of output images, a tensor source ----
def _same_images(srcs, dtype):
    p0, w, h, pitch = _image(srcs[0], dtype)
    for s in srcs:
        assert _image(s, dtype)[1:] == (w, h, pitch)
    return (C.c_void_p * len(srcs))(*[s.data_ptr() for s in srcs]), w, h, pitch


def conditional_copy_u8c3(srcs, used, default, out, stream=None, defer=False):
    """srcs: list of (H, W, 3) uint8 of one size/pitch; out: (n, H, W, 3) uint8 contiguous; planes from `used` on receive `default`."""
    _, capi = load()
    ptrs, w, h, pitch = _same_images(srcs, "uint8")
    out = _dev(out, "uint8")
    assert out.shape == (len(srcs), h, w, 3) and out.is_contiguous()
    d = (C.c_uint8 * 3)(*[int(v) for v in default])
    _deferred = _call(capi.fk_conditional_copy_u8c3, (ptrs, w, h, pitch, len(srcs), int(used), d, C.c_void_p(out.data_ptr()), _stream(stream)), defer)
    return _deferred if defer else out


def conditional_resize_f32c3(srcs, used, default, out, stream=None, defer=False):
    """srcs: list of (H, W, 3) uint8 of one size/pitch; out: (n, dst_h, dst_w, 3) float32 contiguous; planes from `used` on receive `default`."""
    _, capi = load()
    ptrs, w, h, pitch = _same_images(srcs, "uint8")
    out = _dev(out, "float32")
    assert out.shape[0] == len(srcs) and out.shape[3] == 3 and out.is_contiguous()
    _deferred = _call(capi.fk_conditional_resize_f32c3, (ptrs, w, h, pitch, len(srcs), int(used), _f3(default), out.shape[2], out.shape[1],
                                                           C.c_void_p(out.data_ptr()), _stream(stream)), defer)
    return _deferred if defer else out


def muladd_midwrite_f32c3(src, mul_v, add_v, mid, out, stream=None, defer=False):
    """src, mid, out: (H, W, 3) float32; mid receives src * mul_v, out receives src * mul_v + add_v."""
    _, capi = load()
    p, w, h, pitch = _image(src, "float32")
    pm, wm, hm, pitch_m = _image(mid, "float32")
    po, wo, ho, pitch_o = _image(out, "float32")
    assert (w, h) == (wm, hm) == (wo, ho)
    _deferred = _call(capi.fk_muladd_midwrite_f32c3, (p, w, h, pitch, mul_v, add_v, pm, pitch_m, po, pitch_o, _stream(stream)), defer)
    return _deferred if defer else (mid, out)


def batch_crop_cast_images(src, rects, outs, stream=None, defer=False):
    """src: (H, W, 3) uint8; rects of one size; outs: list of (rh, rw, 3) float32 images of that size and one pitch."""
    _, capi = load()
    p, w, h, pitch = _image(src, "uint8")
    ptrs, ow, oh, out_pitch = _same_images(outs, "float32")
    assert len(outs) == len(rects)
    _deferred = _call(capi.fk_batch_crop_cast_images, (p, w, h, pitch, _rects(rects), len(rects), ptrs, out_pitch, _stream(stream)), defer)
    return _deferred if defer else outs


def tensor_mul_f32c3(src, mul, out, stream=None, defer=False):
    """src, out: (planes, H, W, 3) float32 contiguous."""
    _, capi = load()
    src, out = _dev(src, "float32"), _dev(out, "float32")
    assert src.shape == out.shape and src.shape[3] == 3 and src.is_contiguous() and out.is_contiguous()
    planes, h, w, _ = src.shape
    _deferred = _call(capi.fk_tensor_mul_f32c3, (C.c_void_p(src.data_ptr()), w, h, planes, _f3(mul), C.c_void_p(out.data_ptr()), _stream(stream)), defer)
    return _deferred if defer else out


def set_to_f32c3_tensor(value, out, stream=None, defer=False):
    """fk::setTo on a tensor of packed float3. out: (planes, H, W, 3) float32 contiguous."""
    _, capi = load()
    out = _dev(out, "float32")
    assert out.dim() == 4 and out.shape[3] == 3 and out.is_contiguous()
    planes, h, w, _ = out.shape
    _deferred = _call(capi.fk_set_to_f32c3_tensor, (_f3(value), C.c_void_p(out.data_ptr()), w, h, planes, _stream(stream)), defer)
    return _deferred if defer else out
