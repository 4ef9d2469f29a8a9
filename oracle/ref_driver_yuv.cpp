// ref_driver_yuv.cpp — drives the REFERENCE's own headers (its CPU backend, built exactly as they lie under
// /root/reference, nothing copied, no stand-in headers) behind the C signatures of fk_oracle_yuv.h.
//
// TEST INFRASTRUCTURE ONLY.  Built by oracle/Makefile into oracle/_ref/libfkref_yuv.so when the reference tree is
// present; used to validate the C restatement in fk_oracle_yuv.c.
//
// The RawImage handed to the reference describes its buffer with the IMAGE height (data.dims.height = height):
// the reference places the chroma plane of semi-planar formats at pitch * data.dims.height
// (algorithms/image_processing/color_conversion.h:337,353), which is where the chroma rows are only under that
// description.  Resize chains take the reference's host interpolation branch (row index from the x coordinate).
#include <fused_kernel/core/execution_model/memory_operations.h>
#include <fused_kernel/algorithms/basic_ops/arithmetic.h>
#include <fused_kernel/algorithms/image_processing/crop.h>
#include <fused_kernel/algorithms/image_processing/color_conversion.h>
#include <fused_kernel/algorithms/image_processing/resize.h>
#include <fused_kernel/fused_kernel.h>

#include <cstdint>
#include <cstddef>

#include "fk_oracle_yuv.h"

using namespace fk;

namespace {
using CPU = TransformDPP<ParArch::CPU>;

template <PixelFormat PF>
RawImage<PF> raw_image(const void* data, size_t pitch, int w, int h) {
    using Base = typename RawImage<PF>::BaseType;
    const uint data_w = static_cast<uint>(w * PixelFormatTraits<PF>::rf.width_f);
    return RawImage<PF>{ RawPtr<ND::_2D, Base>{ const_cast<Base*>(static_cast<const Base*>(data)),
                                                 PtrDims<ND::_2D>(data_w, static_cast<uint>(h), static_cast<uint>(pitch)) },
                         static_cast<uint>(w), static_cast<uint>(h) };
}
template <typename T>
RawPtr<ND::_2D, T> raw2d(const void* data, int w, int h, size_t pitch) {
    return RawPtr<ND::_2D, T>{ const_cast<T*>(static_cast<const T*>(data)),
                               PtrDims<ND::_2D>(static_cast<uint>(w), static_cast<uint>(h), static_cast<uint>(pitch)) };
}

template <PixelFormat PF>
void read_yuv(const void* src, size_t pitch, int w, int h, void* dst, size_t dst_pitch) {
    using Pixel = typename ReadYUV<PF>::OutputType;
    Stream_<ParArch::CPU> stream;
    executeOperations<CPU>(stream, ReadYUV<PF>::build(raw_image<PF>(src, pitch, w, h)),
                           PerThreadWrite<ND::_2D, Pixel>::build(raw2d<Pixel>(dst, w, h, dst_pitch)));
}
template <PixelFormat PF>
void write_yuv(const void* src, size_t pitch, int w, int h, void* dst, size_t dst_pitch) {
    using Pixel = typename WriteYUV<PF>::InputType;
    Stream_<ParArch::CPU> stream;
    executeOperations<CPU>(stream, PerThreadRead<ND::_2D, Pixel>::build(raw2d<Pixel>(src, w, h, pitch)),
                           WriteYUV<PF>::build(raw_image<PF>(dst, dst_pitch, w, h)));
}
template <PixelFormat PF, ColorRange CR, ColorPrimitives CP, bool ALPHA, bool FLOAT_OUT>
void to_rgb(const void* src, size_t pitch, int w, int h, void* dst, size_t dst_pitch) {
    using Out = std::conditional_t<FLOAT_OUT, VectorType_t<float, ALPHA ? 4 : 3>, YUVOutputPixelType<PF, ALPHA>>;
    Stream_<ParArch::CPU> stream;
    executeOperations<CPU>(stream, ReadYUV<PF>::build(raw_image<PF>(src, pitch, w, h)),
                           ConvertYUVToRGB<PF, CR, CP, ALPHA, Out>::build(),
                           PerThreadWrite<ND::_2D, Out>::build(raw2d<Out>(dst, w, h, dst_pitch)));
}
template <PixelFormat PF, ColorRange CR, ColorPrimitives CP>
void crop_resize(const void* src, size_t pitch, int w, int h, fko_rect crop, int dw, int dh, float div_v, float* out) {
    Stream_<ParArch::CPU> stream;
    const auto rgb = ReadYUV<PF>::build(raw_image<PF>(src, pitch, w, h)).then(ConvertYUVToRGB<PF, CR, CP, false>::build());
    const auto sender = rgb.then(Crop<>::build(Rect(static_cast<uint>(crop.x), static_cast<uint>(crop.y), crop.width, crop.height)))
                            .then(Resize<InterpolationType::INTER_LINEAR>::build(Size(dw, dh)))
                            .then(Div<float3>::build(make_set<float3>(div_v)));
    const RawPtr<ND::_3D, float> planes{ out, PtrDims<ND::_3D>(static_cast<uint>(dw), static_cast<uint>(dh), 1u, 3u,
                                                                static_cast<uint>(sizeof(float) * dw)) };
    executeOperations<CPU>(stream, sender, TensorSplit<float3>::build(planes));
}

#define FKR_FORMAT_SWITCH(format, CALL)                                                                                \
    switch (format) {                                                                                                  \
    case FKO_PF_NV12: { constexpr PixelFormat PF = PixelFormat::NV12; CALL; return 0; }                                \
    case FKO_PF_NV21: { constexpr PixelFormat PF = PixelFormat::NV21; CALL; return 0; }                                \
    case FKO_PF_P010: { constexpr PixelFormat PF = PixelFormat::P010; CALL; return 0; }                                \
    case FKO_PF_P210: { constexpr PixelFormat PF = PixelFormat::P210; CALL; return 0; }                                \
    case FKO_PF_Y210: { constexpr PixelFormat PF = PixelFormat::Y210; CALL; return 0; }                                \
    case FKO_PF_UYVY: { constexpr PixelFormat PF = PixelFormat::UYVY; CALL; return 0; }                                \
    default: return 1;                                                                                                 \
    }

template <PixelFormat PF, bool ALPHA, bool FLOAT_OUT>
int to_rgb_matrix(int range, int primaries, const void* src, size_t pitch, int w, int h, void* dst, size_t dst_pitch) {
    using R = ColorRange;
    using P = ColorPrimitives;
    if (range == FKO_RANGE_FULL && primaries == FKO_BT601) to_rgb<PF, R::Full, P::bt601, ALPHA, FLOAT_OUT>(src, pitch, w, h, dst, dst_pitch);
    else if (range == FKO_RANGE_FULL && primaries == FKO_BT709) to_rgb<PF, R::Full, P::bt709, ALPHA, FLOAT_OUT>(src, pitch, w, h, dst, dst_pitch);
    else if (range == FKO_RANGE_LIMITED && primaries == FKO_BT709) to_rgb<PF, R::Limited, P::bt709, ALPHA, FLOAT_OUT>(src, pitch, w, h, dst, dst_pitch);
    else if (range == FKO_RANGE_FULL && primaries == FKO_BT2020) to_rgb<PF, R::Full, P::bt2020, ALPHA, FLOAT_OUT>(src, pitch, w, h, dst, dst_pitch);
    else return 1;
    return 0;
}
template <PixelFormat PF>
int to_rgb_any(int range, int primaries, int alpha, int float_out, const void* src, size_t pitch, int w, int h, void* dst, size_t dst_pitch) {
    if (alpha && float_out) return to_rgb_matrix<PF, true, true>(range, primaries, src, pitch, w, h, dst, dst_pitch);
    if (alpha) return to_rgb_matrix<PF, true, false>(range, primaries, src, pitch, w, h, dst, dst_pitch);
    if (float_out) return to_rgb_matrix<PF, false, true>(range, primaries, src, pitch, w, h, dst, dst_pitch);
    return to_rgb_matrix<PF, false, false>(range, primaries, src, pitch, w, h, dst, dst_pitch);
}
template <PixelFormat PF>
int crop_resize_any(int range, int primaries, const void* src, size_t pitch, int w, int h, fko_rect crop, int dw, int dh, float div_v, float* out) {
    using R = ColorRange;
    using P = ColorPrimitives;
    if (range == FKO_RANGE_FULL && primaries == FKO_BT601) crop_resize<PF, R::Full, P::bt601>(src, pitch, w, h, crop, dw, dh, div_v, out);
    else if (range == FKO_RANGE_FULL && primaries == FKO_BT709) crop_resize<PF, R::Full, P::bt709>(src, pitch, w, h, crop, dw, dh, div_v, out);
    else if (range == FKO_RANGE_LIMITED && primaries == FKO_BT709) crop_resize<PF, R::Limited, P::bt709>(src, pitch, w, h, crop, dw, dh, div_v, out);
    else if (range == FKO_RANGE_FULL && primaries == FKO_BT2020) crop_resize<PF, R::Full, P::bt2020>(src, pitch, w, h, crop, dw, dh, div_v, out);
    else return 1;
    return 0;
}
} // namespace

extern "C" {

int fkr_read_yuv(int format, const void* src, size_t src_pitch, int width, int height, void* dst, size_t dst_pitch) {
    FKR_FORMAT_SWITCH(format, (read_yuv<PF>(src, src_pitch, width, height, dst, dst_pitch)))
}
int fkr_write_yuv(int format, const void* src, size_t src_pitch, int width, int height, void* dst, size_t dst_pitch) {
    FKR_FORMAT_SWITCH(format, (write_yuv<PF>(src, src_pitch, width, height, dst, dst_pitch)))
}
int fkr_yuv_to_rgb(int format, int range, int primaries, int alpha, int float_out, const void* src, size_t src_pitch,
                   int width, int height, void* dst, size_t dst_pitch) {
    FKR_FORMAT_SWITCH(format, (void)0; return (to_rgb_any<PF>(range, primaries, alpha, float_out, src, src_pitch, width, height, dst, dst_pitch)))
}
int fkr_yuv_crop_resize_norm_split(int format, int range, int primaries, const void* src, size_t src_pitch, int width,
                                   int height, fko_rect crop, int dst_w, int dst_h, float div_v, float* out) {
    FKR_FORMAT_SWITCH(format, (void)0; return (crop_resize_any<PF>(range, primaries, src, src_pitch, width, height, crop, dst_w, dst_h, div_v, out)))
}

} // extern "C"
