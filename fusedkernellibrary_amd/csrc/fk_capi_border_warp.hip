// fk_capi_border_warp.hip — the BorderReader, Warping and Deinterlace entry points of include/fk_capi.h, built with the fk::
// operator API and handed to executeOperations.  Compiled by hipcc into libfk_capi.so.
#include "fk_capi_common.h"

using namespace fk;
using namespace fk_capi;

namespace {

template <BorderType BT>
void border_crop(Stream& stream, const void* src, int w, int h, size_t pitch, int left, int top, int dw, int dh, const uint8_t* value,
                 void* dst, size_t dst_pitch) {
    const auto read = PerThreadRead<ND::_2D, uchar3>::build(view2d<uchar3>(src, w, h, pitch));
    const Rect window(static_cast<uint>(-left), static_cast<uint>(-top), dw, dh);
    const auto write = PerThreadWrite<ND::_2D, uchar3>::build(view2d<uchar3>(dst, dw, dh, dst_pitch));
    if constexpr (BT == BorderType::CONSTANT) {
        executeOperations<TransformDPP<>>(stream, read.then(BorderReader<BT>::build(uchar3{ value[0], value[1], value[2] })).then(Crop<>::build(window)), write);
    } else {
        executeOperations<TransformDPP<>>(stream, read.then(BorderReader<BT>::template build<uchar3>()).then(Crop<>::build(window)), write);
    }
}

template <WarpType WT>
void warp(Stream& stream, const float* m, const void* src, int w, int h, size_t pitch, int dw, int dh, void* dst, size_t dst_pitch) {
    WarpingParameters<WT> params{};
    constexpr int ROWS = WT == WarpType::Affine ? 2 : 3;
    for (int r = 0; r < ROWS; ++r)
        for (int c = 0; c < 3; ++c) params.transformMatrix.data[r][c] = m[3 * r + c];
    params.dstSize = Size(dw, dh);
    const auto sender = PerThreadRead<ND::_2D, uchar3>::build(view2d<uchar3>(src, w, h, pitch)).then(Warping<WT>::build(params));
    executeOperations<TransformDPP<>>(stream, sender, PerThreadWrite<ND::_2D, float3>::build(view2d<float3>(dst, dw, dh, dst_pitch)));
}

} // namespace

extern "C" {

int fk_border_crop_u8c3(int border_type, const void* src, int w, int h, size_t src_pitch, int left, int top, int dst_w, int dst_h,
                        const uint8_t value[3], void* dst, size_t dst_pitch, void* stream) {
    if (src == nullptr || dst == nullptr) return bad_argument("null pointer");
    if (w <= 0 || h <= 0 || dst_w <= 0 || dst_h <= 0) return bad_argument("empty image");
    if (src_pitch < static_cast<size_t>(w) * 3 || dst_pitch < static_cast<size_t>(dst_w) * 3) return bad_argument("pitch shorter than a row");
    if (border_type == FK_BORDER_CONSTANT && value == nullptr) return bad_argument("a constant border needs its value");
    return guarded([&]() -> int {
        Stream s(stream);
        switch (border_type) {
        case FK_BORDER_CONSTANT: border_crop<BorderType::CONSTANT>(s, src, w, h, src_pitch, left, top, dst_w, dst_h, value, dst, dst_pitch); break;
        case FK_BORDER_REPLICATE: border_crop<BorderType::REPLICATE>(s, src, w, h, src_pitch, left, top, dst_w, dst_h, value, dst, dst_pitch); break;
        case FK_BORDER_REFLECT: border_crop<BorderType::REFLECT>(s, src, w, h, src_pitch, left, top, dst_w, dst_h, value, dst, dst_pitch); break;
        case FK_BORDER_WRAP: border_crop<BorderType::WRAP>(s, src, w, h, src_pitch, left, top, dst_w, dst_h, value, dst, dst_pitch); break;
        case FK_BORDER_REFLECT_101: border_crop<BorderType::REFLECT_101>(s, src, w, h, src_pitch, left, top, dst_w, dst_h, value, dst, dst_pitch); break;
        default: return unsupported("border type not implemented (CONSTANT, REPLICATE, REFLECT, WRAP, REFLECT_101)");
        }
        return FK_OK;
    });
}

int fk_warp_u8c3_f32c3(int warp_type, const float* matrix, const void* src, int w, int h, size_t src_pitch, int dst_w, int dst_h,
                       void* dst, size_t dst_pitch, void* stream) {
    if (src == nullptr || dst == nullptr || matrix == nullptr) return bad_argument("null pointer");
    if (w <= 0 || h <= 0 || dst_w <= 0 || dst_h <= 0) return bad_argument("empty image");
    if (src_pitch < static_cast<size_t>(w) * 3 || dst_pitch < static_cast<size_t>(dst_w) * 12) return bad_argument("pitch shorter than a row");
    if (!interpolation_rows_exist(0, w, h)) return rows_missing();
    return guarded([&]() -> int {
        Stream s(stream);
        if (warp_type == FK_WARP_AFFINE) warp<WarpType::Affine>(s, matrix, src, w, h, src_pitch, dst_w, dst_h, dst, dst_pitch);
        else if (warp_type == FK_WARP_PERSPECTIVE) warp<WarpType::Perspective>(s, matrix, src, w, h, src_pitch, dst_w, dst_h, dst, dst_pitch);
        else return unsupported("warp type must be affine or perspective");
        return FK_OK;
    });
}

int fk_deinterlace_u8c3_f32c3(int type, int use_even_lines, const void* src, int w, int h, size_t src_pitch, void* dst, size_t dst_pitch,
                              void* stream) {
    if (src == nullptr || dst == nullptr) return bad_argument("null pointer");
    if (w <= 0 || h <= 0) return bad_argument("empty image");
    if (src_pitch < static_cast<size_t>(w) * 3 || dst_pitch < static_cast<size_t>(w) * 12) return bad_argument("pitch shorter than a row");
    return guarded([&]() -> int {
        Stream s(stream);
        const auto read = PerThreadRead<ND::_2D, uchar3>::build(view2d<uchar3>(src, w, h, src_pitch));
        const auto write = PerThreadWrite<ND::_2D, float3>::build(view2d<float3>(dst, w, h, dst_pitch));
        if (type == FK_DEINTERLACE_BLEND) {
            executeOperations<TransformDPP<>>(s, read.then(Deinterlace<DeinterlaceType::BLEND>::build()), write);
        } else if (type == FK_DEINTERLACE_INTER_LINEAR) {
            const DeinterlaceParameters<DeinterlaceType::INTER_LINEAR> params{ use_even_lines != 0 };
            executeOperations<TransformDPP<>>(s, read.then(Deinterlace<DeinterlaceType::INTER_LINEAR>::build(params)), write);
        } else {
            return unsupported("deinterlace type must be BLEND or INTER_LINEAR");
        }
        return FK_OK;
    });
}

} // extern "C"
