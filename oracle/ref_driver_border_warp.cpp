// ref_driver_border_warp.cpp — drives the REFERENCE's own headers (its CPU backend, built exactly as they lie under
// /root/reference, nothing copied, no stand-in headers) behind the C signatures of fk_oracle_border_warp.h.
//
// TEST INFRASTRUCTURE ONLY.  Built by oracle/Makefile into oracle/_ref/libfkref_border_warp.so when the reference
// tree is present.  Warping takes the reference's host interpolation branch (row index from the x coordinate);
// callers keep source images at least as tall as they are wide so that it stays in bounds.
#include <fused_kernel/core/execution_model/memory_operations.h>
#include <fused_kernel/algorithms/image_processing/border_reader.h>
#include <fused_kernel/algorithms/image_processing/crop.h>
#include <fused_kernel/algorithms/image_processing/deinterlace.h>
#include <fused_kernel/algorithms/image_processing/warping.h>
#include <fused_kernel/fused_kernel.h>

#include <cstdint>
#include <cstddef>

#include "fk_oracle_border_warp.h"

using namespace fk;

namespace {
using CPU = TransformDPP<ParArch::CPU>;

template <typename T>
RawPtr<ND::_2D, T> raw2d(const void* data, int w, int h, size_t pitch) {
    return RawPtr<ND::_2D, T>{ const_cast<T*>(static_cast<const T*>(data)),
                               PtrDims<ND::_2D>(static_cast<uint>(w), static_cast<uint>(h), static_cast<uint>(pitch)) };
}

template <BorderType BT>
void border_crop(const uint8_t* src, int w, int h, size_t pitch, int left, int top, int dw, int dh, const uint8_t* value,
                 uint8_t* dst, size_t dst_pitch) {
    Stream_<ParArch::CPU> stream;
    const auto read = PerThreadRead<ND::_2D, uchar3>::build(raw2d<uchar3>(src, w, h, pitch));
    const Rect window(static_cast<uint>(-left), static_cast<uint>(-top), dw, dh);
    const auto write = PerThreadWrite<ND::_2D, uchar3>::build(raw2d<uchar3>(dst, dw, dh, dst_pitch));
    // the complete forms are named directly: the reference's entry form BorderReader<BT>::build(readIOp) is ambiguous
    // for the border types without a value
    using ReadIOp = std::decay_t<decltype(read)>;
    if constexpr (BT == BorderType::CONSTANT) {
        const auto bordered = BorderReader<BT, ReadIOp>::build(read, uchar3{ value[0], value[1], value[2] });
        executeOperations<CPU>(stream, Crop<std::decay_t<decltype(bordered)>>::build(bordered, window), write);
    } else {
        const auto bordered = BorderReader<BT, ReadIOp>::build(read);
        executeOperations<CPU>(stream, Crop<std::decay_t<decltype(bordered)>>::build(bordered, window), write);
    }
}

template <WarpType WT>
void warp(const float* m, const uint8_t* src, int w, int h, size_t pitch, int dw, int dh, float* dst, size_t dst_pitch) {
    Stream_<ParArch::CPU> stream;
    WarpingParameters<WT> params{};
    constexpr int ROWS = WT == WarpType::Affine ? 2 : 3;
    for (int r = 0; r < ROWS; ++r)
        for (int c = 0; c < 3; ++c) params.transformMatrix.data[r][c] = m[3 * r + c];
    params.dstSize = Size(dw, dh);
    const auto sender = PerThreadRead<ND::_2D, uchar3>::build(raw2d<uchar3>(src, w, h, pitch)).then(Warping<WT>::build(params));
    executeOperations<CPU>(stream, sender, PerThreadWrite<ND::_2D, float3>::build(raw2d<float3>(dst, dw, dh, dst_pitch)));
}
} // namespace

extern "C" {

int fkr_border_crop_u8c3(int border_type, const uint8_t* src, int w, int h, size_t src_pitch, int left, int top, int dst_w,
                         int dst_h, const uint8_t* value, uint8_t* dst, size_t dst_pitch) {
    switch (border_type) {
    case FKO_BORDER_CONSTANT: border_crop<BorderType::CONSTANT>(src, w, h, src_pitch, left, top, dst_w, dst_h, value, dst, dst_pitch); return 0;
    case FKO_BORDER_REPLICATE: border_crop<BorderType::REPLICATE>(src, w, h, src_pitch, left, top, dst_w, dst_h, value, dst, dst_pitch); return 0;
    case FKO_BORDER_REFLECT: border_crop<BorderType::REFLECT>(src, w, h, src_pitch, left, top, dst_w, dst_h, value, dst, dst_pitch); return 0;
    case FKO_BORDER_WRAP: border_crop<BorderType::WRAP>(src, w, h, src_pitch, left, top, dst_w, dst_h, value, dst, dst_pitch); return 0;
    case FKO_BORDER_REFLECT_101: border_crop<BorderType::REFLECT_101>(src, w, h, src_pitch, left, top, dst_w, dst_h, value, dst, dst_pitch); return 0;
    default: return 1;
    }
}

void fkr_warp_coords(int warp_type, const float* m, int x, int y, float* out) {
    float2 c;
    if (warp_type == FKO_WARP_PERSPECTIVE) {
        WarpingParameters<WarpType::Perspective> p{};
        for (int r = 0; r < 3; ++r)
            for (int k = 0; k < 3; ++k) p.transformMatrix.data[r][k] = m[3 * r + k];
        c = WarpingCoords<WarpType::Perspective>::exec(Point(x, y), p);
    } else {
        WarpingParameters<WarpType::Affine> p{};
        for (int r = 0; r < 2; ++r)
            for (int k = 0; k < 3; ++k) p.transformMatrix.data[r][k] = m[3 * r + k];
        c = WarpingCoords<WarpType::Affine>::exec(Point(x, y), p);
    }
    out[0] = c.x;
    out[1] = c.y;
}

int fkr_warp_u8c3_f32c3(int warp_type, const float* matrix, const uint8_t* src, int w, int h, size_t src_pitch, int dst_w,
                        int dst_h, float* dst, size_t dst_pitch) {
    if (warp_type == FKO_WARP_AFFINE) warp<WarpType::Affine>(matrix, src, w, h, src_pitch, dst_w, dst_h, dst, dst_pitch);
    else if (warp_type == FKO_WARP_PERSPECTIVE) warp<WarpType::Perspective>(matrix, src, w, h, src_pitch, dst_w, dst_h, dst, dst_pitch);
    else return 1;
    return 0;
}

int fkr_deinterlace_u8c3_f32c3(int type, int use_even_lines, const uint8_t* src, int w, int h, size_t src_pitch, float* dst, size_t dst_pitch) {
    Stream_<ParArch::CPU> stream;
    const auto read = PerThreadRead<ND::_2D, uchar3>::build(raw2d<uchar3>(src, w, h, src_pitch));
    const auto write = PerThreadWrite<ND::_2D, float3>::build(raw2d<float3>(dst, w, h, dst_pitch));
    if (type == FKO_DEINTERLACE_BLEND) {
        executeOperations<CPU>(stream, read.then(Deinterlace<DeinterlaceType::BLEND>::build()), write);
    } else if (type == FKO_DEINTERLACE_INTER_LINEAR) {
        const DeinterlaceParameters<DeinterlaceType::INTER_LINEAR> params{ use_even_lines != 0 };
        executeOperations<CPU>(stream, read.then(Deinterlace<DeinterlaceType::INTER_LINEAR>::build(params)), write);
    } else {
        return 1;
    }
    return 0;
}

} // extern "C"
