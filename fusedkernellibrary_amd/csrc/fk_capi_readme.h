// One plane of the README pipeline (tests/examples/readme_test_code.h:26-72 of the reference) as a fused read, shared by
// the entry points that launch it: PerThreadRead<_2D,uchar3> -> Crop(rect) -> Resize<INTER_LINEAR, AR>(dw x dh,
// background) -> Mul<float3> -> Sub<float3> -> Div<float3> -> ColorConversion<COLOR_RGB2BGR>.
#ifndef FK_CAPI_README_H
#define FK_CAPI_README_H

#include "fk_capi_common.h"

namespace fk_capi {

inline fk::Rect rect_of(const fk_rect& r) { return fk::Rect(static_cast<fk::uint>(r.x), static_cast<fk::uint>(r.y), r.width, r.height); }
inline fk::float3 f3(const float* v) { return fk::float3{ v[0], v[1], v[2] }; }
inline bool rects_inside(const fk_rect* r, int n, int w, int h) {
    for (int i = 0; i < n; ++i) {
        if (r[i].x < 0 || r[i].y < 0 || r[i].width <= 0 || r[i].height <= 0 || r[i].x + r[i].width > w || r[i].y + r[i].height > h) return false;
    }
    return true;
}

template <fk::AspectRatio AR>
auto readme_plane(const void* src, int w, int h, size_t pitch, const fk_rect& rect, int dw, int dh, const float* bg, const float* mul,
                  const float* sub, const float* div) {
    using namespace fk;
    const auto cropped = PerThreadRead<ND::_2D, uchar3>::build(view2d<uchar3>(src, w, h, pitch)).then(Crop<>::build(rect_of(rect)));
    const auto finish = [&](const auto& resized) {
        return resized.then(Mul<float3>::build(f3(mul)))
            .then(Sub<float3>::build(f3(sub)))
            .then(Div<float3>::build(f3(div)))
            .then(ColorConversion<ColorConversionCodes::COLOR_RGB2BGR, float3, float3>::build());
    };
    if constexpr (AR == AspectRatio::IGNORE_AR) {
        return finish(cropped.then(Resize<InterpolationType::INTER_LINEAR, AR>::build(Size(dw, dh))));
    } else {
        return finish(cropped.then(Resize<InterpolationType::INTER_LINEAR, AR>::build(Size(dw, dh), f3(bg))));
    }
}

// the checks that the entry points of this pipeline share; FK_OK when the arguments are usable
inline int check_readme_arguments(const void* src, int src_w, int src_h, const fk_rect* rects, int n, int dst_w, int dst_h, const float* out) {
    if (src == nullptr || out == nullptr || rects == nullptr || dst_w <= 0 || dst_h <= 0 || n <= 0) return bad_argument("null pointer, empty destination or no planes");
    if (!rects_inside(rects, n, src_w, src_h)) return bad_argument("crop rectangle outside the source image");
    for (int i = 0; i < n; ++i) {
        if (!interpolation_rows_exist(rects[i].y, rects[i].width, src_h)) return rows_missing();
    }
    return FK_OK;
}

} // namespace fk_capi
#endif
