// fk_capi.hip — the C entry points of include/fk_capi.h: each builds its chain with the fk:: operator API
// (PerThreadRead(...).then(...)..., TensorWrite) and hands it to executeOperations, which instantiates the fused
// gfx950 kernel for that chain.  Compiled by hipcc into libfk_capi.so.
#include <array>
#include <vector>

#include "fk_capi_readme.h"

using namespace fk;
using namespace fk_capi;

namespace fk_capi {
std::string& last_error() {
    thread_local std::string text;
    return text;
}
} // namespace fk_capi

namespace {
using Linear = InterpolationType;

// A batch of n planes, n known at run time: the planes are built one by one with the same .then() chain (what the
// batch builders of the operator API do per element of their arrays), put into batch reads of a fixed capacity with n of
// their entries in use, and launched 64 planes at a time; `receiver_for(first, count)` builds the write for planes
// first .. first + count - 1.  The plane table travels in the kernel-argument segment like that of a batch whose size is
// a template argument.  Every launch gets the thread grid of the whole batch (the largest width and height among all n
// planes, batch_operations.h:153-160), so that what a plane holds beside its own window does not depend on which launch
// it falls in.
constexpr size_t SMALL_BATCH = 8, LARGE_BATCH = 64;
template <typename PlaneIOp, typename ReceiverFor>
void launch_planes(Stream& stream, const std::vector<PlaneIOp>& planes, const ReceiverFor& receiver_for) {
    using Op = typename PlaneIOp::Operation;
    uint box_w = 0, box_h = 0;
    for (const PlaneIOp& plane : planes) {
        const uint w = Op::num_elems_x(Point(0, 0, 0), plane), h = Op::num_elems_y(Point(0, 0, 0), plane);
        box_w = w > box_w ? w : box_w;
        box_h = h > box_h ? h : box_h;
    }
    for (size_t first = 0; first < planes.size(); first += LARGE_BATCH) {
        const size_t count = planes.size() - first < LARGE_BATCH ? planes.size() - first : LARGE_BATCH;
        if (count <= SMALL_BATCH) {
            executeOperations<TransformDPP<>>(stream, BatchRead<SMALL_BATCH>::build_first(&planes[first], count, box_w, box_h), receiver_for(first, count));
        } else {
            executeOperations<TransformDPP<>>(stream, BatchRead<LARGE_BATCH>::build_first(&planes[first], count, box_w, box_h), receiver_for(first, count));
        }
    }
}

template <AspectRatio AR>
void readme_pipeline(Stream& stream, const void* src, int w, int h, size_t pitch, const fk_rect* rects, int n, int dw, int dh,
                     const float* bg, const float* mul, const float* sub, const float* div, float* out) {
    std::vector<decltype(readme_plane<AR>(src, w, h, pitch, rects[0], dw, dh, bg, mul, sub, div))> planes;
    for (int i = 0; i < n; ++i) planes.push_back(readme_plane<AR>(src, w, h, pitch, rects[i], dw, dh, bg, mul, sub, div));
    const size_t plane_floats = static_cast<size_t>(dw) * dh * 3;
    launch_planes(stream, planes, [&](size_t first, size_t count) {
        return TensorWrite<float3>::build(view3d<float3>(out + first * plane_floats, dw, dh, static_cast<int>(count), 1));
    });
}

int readme_pipeline_any_ar(Stream& stream, int aspect, const void* src, int w, int h, size_t pitch, const fk_rect* rects, int n, int dw,
                           int dh, const float* bg, const float* mul, const float* sub, const float* div, float* out) {
    switch (aspect) {
    case FK_PRESERVE_AR: readme_pipeline<AspectRatio::PRESERVE_AR>(stream, src, w, h, pitch, rects, n, dw, dh, bg, mul, sub, div, out); return FK_OK;
    case FK_IGNORE_AR: readme_pipeline<AspectRatio::IGNORE_AR>(stream, src, w, h, pitch, rects, n, dw, dh, bg, mul, sub, div, out); return FK_OK;
    case FK_PRESERVE_AR_RN_EVEN: readme_pipeline<AspectRatio::PRESERVE_AR_RN_EVEN>(stream, src, w, h, pitch, rects, n, dw, dh, bg, mul, sub, div, out); return FK_OK;
    case FK_PRESERVE_AR_LEFT: readme_pipeline<AspectRatio::PRESERVE_AR_LEFT>(stream, src, w, h, pitch, rects, n, dw, dh, bg, mul, sub, div, out); return FK_OK;
    default: return unsupported("unknown aspect-ratio mode");
    }
}

void split_pipeline(Stream& stream, const void* const* srcs, int w, int h, size_t pitch, const fk_rect* rects, int n, int dw, int dh,
                    const float* d1, const float* s, const float* d2, float* out) {
    const auto plane = [&](const void* src, const fk_rect& r) {
        return PerThreadRead<ND::_2D, uchar3>::build(view2d<uchar3>(src, w, h, pitch))
            .then(Crop<>::build(rect_of(r)))
            .then(Resize<Linear::INTER_LINEAR>::build(Size(dw, dh)))
            .then(Div<float3>::build(f3(d1)))
            .then(Sub<float3>::build(f3(s)))
            .then(Div<float3>::build(f3(d2)))
            .then(ColorConversion<ColorConversionCodes::COLOR_RGB2BGR, float3, float3>::build());
    };
    std::vector<decltype(plane(srcs[0], rects[0]))> planes;
    for (int i = 0; i < n; ++i) planes.push_back(plane(srcs[i], rects[i]));
    const size_t plane_floats = static_cast<size_t>(dw) * dh * 3;
    launch_planes(stream, planes, [&](size_t first, size_t count) {
        return TensorSplit<float3>::build(view3d<float>(out + first * plane_floats, dw, dh, static_cast<int>(count), 3));
    });
}

void tiles_pipeline(Stream& stream, const void* src, int w, int h, size_t pitch, int rw, int rh, const fk_rect* rects, int n, int tw,
                    int th, const float* mul, float* out) {
    const auto resized = PerThreadRead<ND::_2D, uchar3>::build(view2d<uchar3>(src, w, h, pitch)).then(Resize<Linear::INTER_LINEAR>::build(Size(rw, rh)));
    const auto plane = [&](const fk_rect& r) { return resized.then(Crop<>::build(rect_of(r))).then(Mul<float3>::build(f3(mul))); };
    std::vector<decltype(plane(rects[0]))> planes;
    for (int i = 0; i < n; ++i) planes.push_back(plane(rects[i]));
    const size_t plane_floats = static_cast<size_t>(tw) * th * 3;
    launch_planes(stream, planes, [&](size_t first, size_t count) {
        return TensorWrite<float3>::build(view3d<float3>(out + first * plane_floats, tw, th, static_cast<int>(count), 1));
    });
}

void crops_pipeline(Stream& stream, const void* src, int w, int h, size_t pitch, const fk_rect* rects, int n, int mw, int mh, float* out) {
    const auto read = PerThreadRead<ND::_2D, uchar3>::build(view2d<uchar3>(src, w, h, pitch));
    const auto plane = [&](const fk_rect& r) { return read.then(Crop<>::build(rect_of(r))).then(Cast<uchar3, float3>::build()); };
    std::vector<decltype(plane(rects[0]))> planes;
    for (int i = 0; i < n; ++i) planes.push_back(plane(rects[i]));
    const size_t plane_floats = static_cast<size_t>(mw) * mh * 3;
    launch_planes(stream, planes, [&](size_t first, size_t count) {
        return TensorWrite<float3>::build(view3d<float3>(out + first * plane_floats, mw, mh, static_cast<int>(count), 1));
    });
}

void windows_pipeline(Stream& stream, const void* src, int w, int h, size_t pitch, const fk_rect* rects, int n, float mul_v, float sub_v, float div_v,
                      float* out) {
    const auto read = PerThreadRead<ND::_2D, uchar>::build(view2d<uchar>(src, w, h, pitch));
    const auto plane = [&](const fk_rect& r) {
        return read.then(Crop<>::build(rect_of(r)))
            .then(SaturateCast<uchar, float>::build())
            .then(Mul<float>::build(mul_v))
            .then(Sub<float>::build(sub_v))
            .then(Div<float>::build(div_v));
    };
    std::vector<decltype(plane(rects[0]))> planes;
    for (int i = 0; i < n; ++i) planes.push_back(plane(rects[i]));
    const int rw = rects[0].width, rh = rects[0].height;
    const size_t plane_floats = static_cast<size_t>(rw) * rh;
    launch_planes(stream, planes, [&](size_t first, size_t count) {
        return TensorWrite<float>::build(view3d<float>(out + first * plane_floats, rw, rh, static_cast<int>(count), 1));
    });
}

// read -> Mul -> Add -> Mul -> ... (DEPTH operations) -> write, built one .then() at a time
template <int DEPTH, int K = 0, typename Sender, typename Receiver>
void muladd_chain(Stream& stream, const Sender& sender, float mul_v, float add_v, const Receiver& receiver) {
    if constexpr (K == DEPTH) {
        executeOperations<TransformDPP<>>(stream, sender, receiver);
    } else if constexpr (K % 2 == 0) {
        muladd_chain<DEPTH, K + 1>(stream, sender.then(Mul<float3>::build(make_set<float3>(mul_v))), mul_v, add_v, receiver);
    } else {
        muladd_chain<DEPTH, K + 1>(stream, sender.then(Add<float3>::build(make_set<float3>(add_v))), mul_v, add_v, receiver);
    }
}

// The four chains of the divergent launch as operation sequences.
auto gray_sequence(const void* src, int w, int h, size_t pitch, void* dst, size_t dst_pitch) {
    return buildOperationSequence(PerThreadRead<ND::_2D, uchar4>::build(view2d<uchar4>(src, w, h, pitch)),
                                  ColorConversion<ColorConversionCodes::COLOR_RGBA2GRAY, uchar4, uchar>::build(),
                                  PerThreadWrite<ND::_2D, uchar>::build(view2d<uchar>(dst, w, h, dst_pitch)));
}
auto resize_sequence(const void* src, int w, int h, size_t pitch, int dw, int dh, float mul_v, void* dst, size_t dst_pitch) {
    return buildOperationSequence(PerThreadRead<ND::_2D, uchar4>::build(view2d<uchar4>(src, w, h, pitch))
                                      .then(Resize<Linear::INTER_LINEAR>::build(Size(dw, dh))),
                                  Mul<float4>::build(make_set<float4>(mul_v)),
                                  PerThreadWrite<ND::_2D, float4>::build(view2d<float4>(dst, dw, dh, dst_pitch)));
}
auto crop_sequence(const void* src, int w, int h, size_t pitch, fk_rect r, int mul_v, void* dst, size_t dst_pitch) {
    return buildOperationSequence(PerThreadRead<ND::_2D, uchar4>::build(view2d<uchar4>(src, w, h, pitch))
                                      .then(Crop<>::build(Rect(static_cast<uint>(r.x), static_cast<uint>(r.y), r.width, r.height))),
                                  Mul<uchar4, int, int4>::build(mul_v), SaturateCast<int4, uchar4>::build(),
                                  PerThreadWrite<ND::_2D, uchar4>::build(view2d<uchar4>(dst, r.width, r.height, dst_pitch)));
}
auto bgr_sequence(const void* src, int w, int h, size_t pitch, float sub_v, void* dst, size_t dst_pitch) {
    return buildOperationSequence(PerThreadRead<ND::_2D, uchar4>::build(view2d<uchar4>(src, w, h, pitch)),
                                  ColorConversion<ColorConversionCodes::COLOR_RGBA2BGR, uchar4, uchar3>::build(),
                                  Cast<uchar3, float3>::build(), Sub<float3>::build(make_set<float3>(sub_v)),
                                  PerThreadWrite<ND::_2D, float3>::build(view2d<float3>(dst, w, h, dst_pitch)));
}
template <typename Sequence>
void run_sequence(Stream& stream, const Sequence& seq) {
    executeOperations<TransformDPP<>>(stream, seq.sender, seq.receiver);
}
} // namespace

extern "C" {

const char* fk_last_error(void) { return last_error().c_str(); }

int fk_interpolate_y1_from_x(void) {
#ifdef FK_INTERPOLATE_Y1_FROM_X
    return 1;
#else
    return 0;
#endif
}

int fk_crop_resize_muls_bgr_tensor(const void* src, int src_w, int src_h, size_t src_pitch, const fk_rect* rects, int n, int dst_w,
                                   int dst_h, int aspect, const float background[3], const float mul[3], const float sub[3],
                                   const float div[3], float* out, void* stream) {
    if (const int rc = check_readme_arguments(src, src_w, src_h, rects, n, dst_w, dst_h, out)) return rc;
    return guarded([&]() -> int {
        Stream s(stream);
        return readme_pipeline_any_ar(s, aspect, src, src_w, src_h, src_pitch, rects, n, dst_w, dst_h, background, mul, sub, div, out);
    });
}

int fk_muladd_chain_f32c3(const void* src, int w, int h, size_t src_pitch, int depth, float mul_v, float add_v, void* dst,
                          size_t dst_pitch, void* stream) {
    if (src == nullptr || dst == nullptr || w <= 0 || h <= 0) return bad_argument("null pointer or empty image");
    return guarded([&]() -> int {
        Stream s(stream);
        const auto read = PerThreadRead<ND::_2D, float3>::build(view2d<float3>(src, w, h, src_pitch));
        const auto write = PerThreadWrite<ND::_2D, float3>::build(view2d<float3>(dst, w, h, dst_pitch));
        switch (depth) {
        case 1: muladd_chain<1>(s, read, mul_v, add_v, write); break;
        case 2: muladd_chain<2>(s, read, mul_v, add_v, write); break;
        case 4: muladd_chain<4>(s, read, mul_v, add_v, write); break;
        case 8: muladd_chain<8>(s, read, mul_v, add_v, write); break;
        case 16: muladd_chain<16>(s, read, mul_v, add_v, write); break;
        case 32: muladd_chain<32>(s, read, mul_v, add_v, write); break;
        case 64: muladd_chain<64>(s, read, mul_v, add_v, write); break;
        case 128: muladd_chain<128>(s, read, mul_v, add_v, write); break;
        default: return unsupported("depth has no instantiation (1, 2, 4, 8, 16, 32, 64, 128)");
        }
        return FK_OK;
    });
}

int fk_single_op_f32c3(const void* src, int w, int h, size_t src_pitch, int is_add, float v, void* dst, size_t dst_pitch, void* stream) {
    if (src == nullptr || dst == nullptr || w <= 0 || h <= 0) return bad_argument("null pointer or empty image");
    return guarded([&]() -> int {
        Stream s(stream);
        const auto read = PerThreadRead<ND::_2D, float3>::build(view2d<float3>(src, w, h, src_pitch));
        const auto write = PerThreadWrite<ND::_2D, float3>::build(view2d<float3>(dst, w, h, dst_pitch));
        if (is_add != 0) executeOperations<TransformDPP<>>(s, read, Add<float3>::build(make_set<float3>(v)), write);
        else executeOperations<TransformDPP<>>(s, read, Mul<float3>::build(make_set<float3>(v)), write);
        return FK_OK;
    });
}

int fk_batch_crop_resize_norm_split(const void* const* srcs, int src_w, int src_h, size_t src_pitch, const fk_rect* rects, int n,
                                    int dst_w, int dst_h, const float div1[3], const float sub[3], const float div2[3], float* out,
                                    void* stream) {
    if (srcs == nullptr || out == nullptr || rects == nullptr || dst_w <= 0 || dst_h <= 0 || n <= 0) return bad_argument("null pointer, empty destination or no planes");
    if (!rects_inside(rects, n, src_w, src_h)) return bad_argument("crop rectangle outside the source image");
    for (int i = 0; i < n; ++i) {
        if (!interpolation_rows_exist(rects[i].y, rects[i].width, src_h)) return rows_missing();
    }
    return guarded([&]() -> int {
        Stream s(stream);
        split_pipeline(s, srcs, src_w, src_h, src_pitch, rects, n, dst_w, dst_h, div1, sub, div2, out);
        return FK_OK;
    });
}

int fk_resize_crop_tiles(const void* src, int src_w, int src_h, size_t src_pitch, int rs_w, int rs_h, const fk_rect* rects, int n,
                         int tile_w, int tile_h, const float mul[3], float* out, void* stream) {
    if (src == nullptr || out == nullptr || rects == nullptr || rs_w <= 0 || rs_h <= 0 || n <= 0) return bad_argument("null pointer, empty destination or no planes");
    if (!rects_inside(rects, n, rs_w, rs_h)) return bad_argument("tile outside the resized image");
    if (!interpolation_rows_exist(0, src_w, src_h)) return rows_missing();
    for (int i = 0; i < n; ++i) {
        if (rects[i].width != tile_w || rects[i].height != tile_h) return bad_argument("every tile must be tile_w x tile_h");
    }
    return guarded([&]() -> int {
        Stream s(stream);
        tiles_pipeline(s, src, src_w, src_h, src_pitch, rs_w, rs_h, rects, n, tile_w, tile_h, mul, out);
        return FK_OK;
    });
}

int fk_rgba2gray_u8c4(const void* src, int w, int h, size_t src_pitch, void* dst, size_t dst_pitch, void* stream) {
    if (src == nullptr || dst == nullptr || w <= 0 || h <= 0) return bad_argument("null pointer or empty image");
    return guarded([&]() -> int {
        Stream s(stream);
        run_sequence(s, gray_sequence(src, w, h, src_pitch, dst, dst_pitch));
        return FK_OK;
    });
}
int fk_resize_mul_u8c4_f32c4(const void* src, int w, int h, size_t src_pitch, int dst_w, int dst_h, float mul_v, void* dst,
                             size_t dst_pitch, void* stream) {
    if (src == nullptr || dst == nullptr || w <= 0 || h <= 0 || dst_w <= 0 || dst_h <= 0) return bad_argument("null pointer or empty image");
    if (!interpolation_rows_exist(0, w, h)) return rows_missing();
    return guarded([&]() -> int {
        Stream s(stream);
        run_sequence(s, resize_sequence(src, w, h, src_pitch, dst_w, dst_h, mul_v, dst, dst_pitch));
        return FK_OK;
    });
}
int fk_crop_mul_saturate_u8c4(const void* src, int w, int h, size_t src_pitch, fk_rect rect, int mul_v, void* dst, size_t dst_pitch,
                              void* stream) {
    if (src == nullptr || dst == nullptr) return bad_argument("null pointer");
    if (!rects_inside(&rect, 1, w, h)) return bad_argument("crop rectangle outside the source image");
    return guarded([&]() -> int {
        Stream s(stream);
        run_sequence(s, crop_sequence(src, w, h, src_pitch, rect, mul_v, dst, dst_pitch));
        return FK_OK;
    });
}
int fk_rgba2bgr_sub_u8c4_f32c3(const void* src, int w, int h, size_t src_pitch, float sub_v, void* dst, size_t dst_pitch, void* stream) {
    if (src == nullptr || dst == nullptr || w <= 0 || h <= 0) return bad_argument("null pointer or empty image");
    return guarded([&]() -> int {
        Stream s(stream);
        run_sequence(s, bgr_sequence(src, w, h, src_pitch, sub_v, dst, dst_pitch));
        return FK_OK;
    });
}

int fk_divergent4_u8c4(const void* src, int w, int h, size_t src_pitch, void* gray_out, int rs_w, int rs_h, float mul_b,
                       void* resized_out, fk_rect rect_c, int mul_c, void* crop_out, float sub_d, void* bgr_out, void* stream) {
    if (src == nullptr || gray_out == nullptr || resized_out == nullptr || crop_out == nullptr || bgr_out == nullptr || w <= 0 || h <= 0 ||
        rs_w <= 0 || rs_h <= 0) {
        return bad_argument("null pointer or empty image");
    }
    if (!rects_inside(&rect_c, 1, w, h)) return bad_argument("crop rectangle outside the source image");
    if (!interpolation_rows_exist(0, w, h)) return rows_missing();
    return guarded([&]() -> int {
        Stream s(stream);
        executeOperations<DivergentBatchTransformDPP<>>(
            s, gray_sequence(src, w, h, src_pitch, gray_out, static_cast<size_t>(w)),
            resize_sequence(src, w, h, src_pitch, rs_w, rs_h, mul_b, resized_out, static_cast<size_t>(rs_w) * sizeof(float4)),
            crop_sequence(src, w, h, src_pitch, rect_c, mul_c, crop_out, static_cast<size_t>(rect_c.width) * sizeof(uchar4)),
            bgr_sequence(src, w, h, src_pitch, sub_d, bgr_out, static_cast<size_t>(w) * sizeof(float3)));
        return FK_OK;
    });
}

int fk_batch_crop_cast_tensor(const void* src, int src_w, int src_h, size_t src_pitch, const fk_rect* rects, int n, int max_w,
                              int max_h, float* out, void* stream) {
    if (src == nullptr || out == nullptr || rects == nullptr || n <= 0) return bad_argument("null pointer or no planes");
    if (!rects_inside(rects, n, src_w, src_h)) return bad_argument("crop rectangle outside the source image");
    for (int i = 0; i < n; ++i) {
        if (rects[i].width > max_w || rects[i].height > max_h) return bad_argument("crop larger than the tensor plane");
    }
    return guarded([&]() -> int {
        Stream s(stream);
        crops_pipeline(s, src, src_w, src_h, src_pitch, rects, n, max_w, max_h, out);
        return FK_OK;
    });
}

int fk_batch_windows_saturate_muls_f32(const void* src, int src_w, int src_h, size_t src_pitch, const fk_rect* rects, int n, float mul_v,
                                       float sub_v, float div_v, float* out, void* stream) {
    if (src == nullptr || out == nullptr || rects == nullptr || n <= 0) return bad_argument("null pointer or no planes");
    if (!rects_inside(rects, n, src_w, src_h)) return bad_argument("window outside the source image");
    for (int i = 0; i < n; ++i) {
        if (rects[i].width != rects[0].width || rects[i].height != rects[0].height) return bad_argument("every window must have the size of the first");
    }
    return guarded([&]() -> int {
        Stream s(stream);
        windows_pipeline(s, src, src_w, src_h, src_pitch, rects, n, mul_v, sub_v, div_v, out);
        return FK_OK;
    });
}

} // extern "C"
