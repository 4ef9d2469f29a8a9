// fk_capi_yuv.hip — the YUV entry points of include/fk_capi.h: ReadYUV / WriteYUV / ConvertYUVToRGB chains built
// with the fk:: operator API and handed to executeOperations.  Compiled by hipcc into libfk_capi.so.
#include "fk_capi_common.h"

using namespace fk;
using namespace fk_capi;

namespace {

template <PixelFormat PF>
RawImage<PF> raw_image(const void* data, size_t pitch, int w, int h) {
    using Base = typename RawImage<PF>::BaseType;
    constexpr ResolutionFactors rf = PixelFormatTraits<PF>::rf;
    return RawImage<PF>{ view2d<Base>(data, static_cast<int>(w * rf.width_f), static_cast<int>(h * rf.height_f), pitch),
                         static_cast<uint>(w), static_cast<uint>(h) };
}

template <PixelFormat PF>
void read_yuv(Stream& stream, const void* src, size_t pitch, int w, int h, void* dst, size_t dst_pitch) {
    using Pixel = typename ReadYUV<PF>::OutputType;
    executeOperations<TransformDPP<>>(stream, ReadYUV<PF>::build(raw_image<PF>(src, pitch, w, h)),
                                      PerThreadWrite<ND::_2D, Pixel>::build(view2d<Pixel>(dst, w, h, dst_pitch)));
}
template <PixelFormat PF>
void write_yuv(Stream& stream, const void* src, size_t pitch, int w, int h, void* dst, size_t dst_pitch) {
    using Pixel = typename WriteYUV<PF>::InputType;
    executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_2D, Pixel>::build(view2d<Pixel>(src, w, h, pitch)),
                                      WriteYUV<PF>::build(raw_image<PF>(dst, dst_pitch, w, h)));
}
template <PixelFormat PF, ColorRange CR, ColorPrimitives CP, bool ALPHA, bool FLOAT_OUT>
void to_rgb(Stream& stream, const void* src, size_t pitch, int w, int h, void* dst, size_t dst_pitch) {
    using Out = std::conditional_t<FLOAT_OUT, VectorType_t<float, ALPHA ? 4 : 3>, YUVOutputPixelType<PF, ALPHA>>;
    executeOperations<TransformDPP<>>(stream, ReadYUV<PF>::build(raw_image<PF>(src, pitch, w, h)),
                                      ConvertYUVToRGB<PF, CR, CP, ALPHA, Out>::build(),
                                      PerThreadWrite<ND::_2D, Out>::build(view2d<Out>(dst, w, h, dst_pitch)));
}
template <PixelFormat PF, ColorRange CR, ColorPrimitives CP>
void crop_resize(Stream& stream, const void* src, size_t pitch, int w, int h, const fk_rect& crop, int dw, int dh, float div_v, float* dst) {
    const auto sender = ReadYUV<PF>::build(raw_image<PF>(src, pitch, w, h))
                            .then(ConvertYUVToRGB<PF, CR, CP, false>::build())
                            .then(Crop<>::build(Rect(static_cast<uint>(crop.x), static_cast<uint>(crop.y), crop.width, crop.height)))
                            .then(Resize<InterpolationType::INTER_LINEAR>::build(Size(dw, dh)))
                            .then(Div<float3>::build(make_set<float3>(div_v)));
    executeOperations<TransformDPP<>>(stream, sender, TensorSplit<float3>::build(view3d<float>(dst, dw, dh, 1, 3)));
}

// CALL sees `PF`; CALL_M additionally `CR` and `CP`
#define FK_FOR_FORMAT(format, CALL)                                                                                    \
    switch (format) {                                                                                                  \
    case FK_PF_NV12: { constexpr PixelFormat PF = PixelFormat::NV12; CALL; break; }                                    \
    case FK_PF_NV21: { constexpr PixelFormat PF = PixelFormat::NV21; CALL; break; }                                    \
    case FK_PF_P010: { constexpr PixelFormat PF = PixelFormat::P010; CALL; break; }                                    \
    case FK_PF_P210: { constexpr PixelFormat PF = PixelFormat::P210; CALL; break; }                                    \
    case FK_PF_Y210: { constexpr PixelFormat PF = PixelFormat::Y210; CALL; break; }                                    \
    case FK_PF_UYVY: { constexpr PixelFormat PF = PixelFormat::UYVY; CALL; break; }                                    \
    default: return unsupported("pixel format not supported (NV12, NV21, P010, P210, Y210, UYVY)");                    \
    }
#define FK_FOR_MATRIX(range, primaries, CALL_M)                                                                        \
    if (range == FK_RANGE_FULL && primaries == FK_BT601) { constexpr ColorRange CR = ColorRange::Full; constexpr ColorPrimitives CP = ColorPrimitives::bt601; CALL_M; } \
    else if (range == FK_RANGE_FULL && primaries == FK_BT709) { constexpr ColorRange CR = ColorRange::Full; constexpr ColorPrimitives CP = ColorPrimitives::bt709; CALL_M; } \
    else if (range == FK_RANGE_LIMITED && primaries == FK_BT709) { constexpr ColorRange CR = ColorRange::Limited; constexpr ColorPrimitives CP = ColorPrimitives::bt709; CALL_M; } \
    else if (range == FK_RANGE_FULL && primaries == FK_BT2020) { constexpr ColorRange CR = ColorRange::Full; constexpr ColorPrimitives CP = ColorPrimitives::bt2020; CALL_M; } \
    else return unsupported("no YCbCr to RGB matrix for this range and primaries");

template <PixelFormat PF, bool ALPHA, bool FLOAT_OUT>
int to_rgb_matrix(Stream& stream, int range, int primaries, const void* src, size_t pitch, int w, int h, void* dst, size_t dst_pitch) {
    FK_FOR_MATRIX(range, primaries, (to_rgb<PF, CR, CP, ALPHA, FLOAT_OUT>(stream, src, pitch, w, h, dst, dst_pitch)))
    return FK_OK;
}
template <PixelFormat PF>
int crop_resize_matrix(Stream& stream, int range, int primaries, const void* src, size_t pitch, int w, int h, const fk_rect& crop,
                       int dw, int dh, float div_v, float* dst) {
    FK_FOR_MATRIX(range, primaries, (crop_resize<PF, CR, CP>(stream, src, pitch, w, h, crop, dw, dh, div_v, dst)))
    return FK_OK;
}

// bytes one image row needs in a raw buffer of this format
size_t raw_row_bytes(int format, int w) {
    switch (format) {
    case FK_PF_NV12: case FK_PF_NV21: return static_cast<size_t>(w);
    case FK_PF_P010: case FK_PF_P210: case FK_PF_UYVY: return 2 * static_cast<size_t>(w);
    case FK_PF_Y210: return 4 * static_cast<size_t>(w);
    default: return 0;
    }
}
size_t base_bytes(int format) { return (format == FK_PF_NV12 || format == FK_PF_NV21 || format == FK_PF_UYVY) ? 1 : 2; }

int check_image(int format, const void* src, const void* dst, int w, int h) {
    if (raw_row_bytes(format, 2) == 0) return unsupported("pixel format not supported (NV12, NV21, P010, P210, Y210, UYVY)");
    if (src == nullptr || dst == nullptr) return bad_argument("null pointer");
    if (w <= 0 || h <= 0 || (w & 1) || (h & 1)) return bad_argument("YUV image width and height must be positive and even");
    return FK_OK;
}
} // namespace

extern "C" {

int fk_read_yuv(int format, const void* src, size_t src_pitch, int width, int height, void* dst, size_t dst_pitch, void* stream) {
    if (const int rc = check_image(format, src, dst, width, height)) return rc;
    if (src_pitch < raw_row_bytes(format, width) || dst_pitch < 3 * base_bytes(format) * width) return bad_argument("pitch shorter than a row");
    return guarded([&]() -> int {
        Stream s(stream);
        FK_FOR_FORMAT(format, (read_yuv<PF>(s, src, src_pitch, width, height, dst, dst_pitch)))
        return FK_OK;
    });
}

int fk_write_yuv(int format, const void* src, size_t src_pitch, int width, int height, void* dst, size_t dst_pitch, void* stream) {
    if (const int rc = check_image(format, src, dst, width, height)) return rc;
    if (dst_pitch < raw_row_bytes(format, width) || src_pitch < 3 * base_bytes(format) * width) return bad_argument("pitch shorter than a row");
    return guarded([&]() -> int {
        Stream s(stream);
        FK_FOR_FORMAT(format, (write_yuv<PF>(s, src, src_pitch, width, height, dst, dst_pitch)))
        return FK_OK;
    });
}

int fk_yuv_to_rgb(int format, int range, int primaries, int alpha, int float_out, const void* src, size_t src_pitch, int width,
                  int height, void* dst, size_t dst_pitch, void* stream) {
    if (const int rc = check_image(format, src, dst, width, height)) return rc;
    const size_t out_pixel = (alpha ? 4 : 3) * (float_out ? sizeof(float) : base_bytes(format));
    if (src_pitch < raw_row_bytes(format, width) || dst_pitch < out_pixel * width) return bad_argument("pitch shorter than a row");
    return guarded([&]() -> int {
        Stream s(stream);
        int rc = FK_OK;
        FK_FOR_FORMAT(format, (rc = alpha ? (float_out ? to_rgb_matrix<PF, true, true>(s, range, primaries, src, src_pitch, width, height, dst, dst_pitch)
                                                       : to_rgb_matrix<PF, true, false>(s, range, primaries, src, src_pitch, width, height, dst, dst_pitch))
                                          : (float_out ? to_rgb_matrix<PF, false, true>(s, range, primaries, src, src_pitch, width, height, dst, dst_pitch)
                                                       : to_rgb_matrix<PF, false, false>(s, range, primaries, src, src_pitch, width, height, dst, dst_pitch))))
        return rc;
    });
}

int fk_yuv_crop_resize_norm_split(int format, int range, int primaries, const void* src, size_t src_pitch, int width, int height,
                                  fk_rect crop, int dst_w, int dst_h, float div_v, float* dst, void* stream) {
    if (const int rc = check_image(format, src, dst, width, height)) return rc;
    if (src_pitch < raw_row_bytes(format, width)) return bad_argument("pitch shorter than a row");
    if (dst_w <= 0 || dst_h <= 0) return bad_argument("empty destination");
    if (crop.x < 0 || crop.y < 0 || crop.width <= 0 || crop.height <= 0 || crop.x + crop.width > width || crop.y + crop.height > height)
        return bad_argument("crop rectangle outside the source image");
    if (!interpolation_rows_exist(crop.y, crop.width, height)) return rows_missing();
    return guarded([&]() -> int {
        Stream s(stream);
        int rc = FK_OK;
        FK_FOR_FORMAT(format, (rc = crop_resize_matrix<PF>(s, range, primaries, src, src_pitch, width, height, crop, dst_w, dst_h, div_v, dst)))
        return rc;
    });
}

} // extern "C"
