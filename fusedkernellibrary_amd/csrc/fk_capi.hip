// fk_capi.hip — the C entry points of include/fk_capi.h: each builds its chain with the fk:: operator API
// (PerThreadRead(...).then(...)..., TensorWrite) and hands it to executeOperations, which instantiates the fused
// gfx950 kernel for that chain.  Compiled by hipcc into libfk_capi.so.
#include <array>

#include "fk_capi_common.h"

using namespace fk;
using namespace fk_capi;

namespace fk_capi {
std::string& last_error() {
    thread_local std::string text;
    return text;
}
} // namespace fk_capi

namespace {
template <size_t N>
std::array<Rect, N> rects_of(const fk_rect* r) {
    std::array<Rect, N> out;
    for (size_t i = 0; i < N; ++i) out[i] = Rect(static_cast<uint>(r[i].x), static_cast<uint>(r[i].y), r[i].width, r[i].height);
    return out;
}
float3 f3(const float* v) { return float3{ v[0], v[1], v[2] }; }

bool rects_inside(const fk_rect* r, int n, int w, int h) {
    for (int i = 0; i < n; ++i) {
        if (r[i].x < 0 || r[i].y < 0 || r[i].width <= 0 || r[i].height <= 0 || r[i].x + r[i].width > w || r[i].y + r[i].height > h) return false;
    }
    return true;
}

using Linear = InterpolationType;

template <size_t N, AspectRatio AR>
void readme_pipeline(Stream& stream, const void* src, int w, int h, size_t pitch, const fk_rect* rects, int dw, int dh,
                     const float* bg, const float* mul, const float* sub, const float* div, float* out) {
    const auto cropped = PerThreadRead<ND::_2D, uchar3>::build(view2d<uchar3>(src, w, h, pitch)).then(Crop<>::build(rects_of<N>(rects)));
    const auto receiver = TensorWrite<float3>::build(view3d<float3>(out, dw, dh, static_cast<int>(N), 1));
    const auto finish = [&](const auto& resized) {
        const auto sender = resized.then(Mul<float3>::build(f3(mul)))
                                .then(Sub<float3>::build(f3(sub)))
                                .then(Div<float3>::build(f3(div)))
                                .then(ColorConversion<ColorConversionCodes::COLOR_RGB2BGR, float3, float3>::build());
        executeOperations<TransformDPP<>>(stream, sender, receiver);
    };
    if constexpr (AR == AspectRatio::IGNORE_AR) {
        finish(cropped.then(Resize<Linear::INTER_LINEAR, AR>::build(Size(dw, dh))));
    } else {
        finish(cropped.then(Resize<Linear::INTER_LINEAR, AR>::build(Size(dw, dh), f3(bg))));
    }
}

template <size_t N>
int readme_pipeline_any_ar(Stream& stream, int aspect, const void* src, int w, int h, size_t pitch, const fk_rect* rects, int dw,
                           int dh, const float* bg, const float* mul, const float* sub, const float* div, float* out) {
    switch (aspect) {
    case FK_PRESERVE_AR: readme_pipeline<N, AspectRatio::PRESERVE_AR>(stream, src, w, h, pitch, rects, dw, dh, bg, mul, sub, div, out); return FK_OK;
    case FK_IGNORE_AR: readme_pipeline<N, AspectRatio::IGNORE_AR>(stream, src, w, h, pitch, rects, dw, dh, bg, mul, sub, div, out); return FK_OK;
    case FK_PRESERVE_AR_RN_EVEN: readme_pipeline<N, AspectRatio::PRESERVE_AR_RN_EVEN>(stream, src, w, h, pitch, rects, dw, dh, bg, mul, sub, div, out); return FK_OK;
    case FK_PRESERVE_AR_LEFT: readme_pipeline<N, AspectRatio::PRESERVE_AR_LEFT>(stream, src, w, h, pitch, rects, dw, dh, bg, mul, sub, div, out); return FK_OK;
    default: return unsupported("unknown aspect-ratio mode");
    }
}

template <size_t N>
void split_pipeline(Stream& stream, const void* const* srcs, int w, int h, size_t pitch, const fk_rect* rects, int dw, int dh,
                    const float* d1, const float* s, const float* d2, float* out) {
    std::array<RawPtr<ND::_2D, uchar3>, N> images;
    for (size_t i = 0; i < N; ++i) images[i] = view2d<uchar3>(srcs[i], w, h, pitch);
    const auto sender = PerThreadRead<ND::_2D, uchar3>::build(images)
                            .then(Crop<>::build(rects_of<N>(rects)))
                            .then(Resize<Linear::INTER_LINEAR>::build(Size(dw, dh)))
                            .then(Div<float3>::build(f3(d1)))
                            .then(Sub<float3>::build(f3(s)))
                            .then(Div<float3>::build(f3(d2)))
                            .then(ColorConversion<ColorConversionCodes::COLOR_RGB2BGR, float3, float3>::build());
    executeOperations<TransformDPP<>>(stream, sender, TensorSplit<float3>::build(view3d<float>(out, dw, dh, static_cast<int>(N), 3)));
}

template <size_t N>
void tiles_pipeline(Stream& stream, const void* src, int w, int h, size_t pitch, int rw, int rh, const fk_rect* rects, int tw,
                    int th, const float* mul, float* out) {
    const auto sender = PerThreadRead<ND::_2D, uchar3>::build(view2d<uchar3>(src, w, h, pitch))
                            .then(Resize<Linear::INTER_LINEAR>::build(Size(rw, rh)))
                            .then(Crop<>::build(rects_of<N>(rects)))
                            .then(Mul<float3>::build(f3(mul)));
    executeOperations<TransformDPP<>>(stream, sender, TensorWrite<float3>::build(view3d<float3>(out, tw, th, static_cast<int>(N), 1)));
}

template <size_t N>
void crops_pipeline(Stream& stream, const void* src, int w, int h, size_t pitch, const fk_rect* rects, int mw, int mh, float* out) {
    const auto sender = PerThreadRead<ND::_2D, uchar3>::build(view2d<uchar3>(src, w, h, pitch))
                            .then(Crop<>::build(rects_of<N>(rects)))
                            .then(Cast<uchar3, float3>::build());
    executeOperations<TransformDPP<>>(stream, sender, TensorWrite<float3>::build(view3d<float3>(out, mw, mh, static_cast<int>(N), 1)));
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

#define FK_FOR_BATCH(n, CALL)                                                                                          \
    switch (n) {                                                                                                       \
    case 1: { constexpr size_t N = 1; CALL; break; }                                                                   \
    case 2: { constexpr size_t N = 2; CALL; break; }                                                                   \
    case 3: { constexpr size_t N = 3; CALL; break; }                                                                   \
    case 5: { constexpr size_t N = 5; CALL; break; }                                                                   \
    case 8: { constexpr size_t N = 8; CALL; break; }                                                                   \
    case 32: { constexpr size_t N = 32; CALL; break; }                                                                 \
    case 50: { constexpr size_t N = 50; CALL; break; }                                                                 \
    default: return unsupported("batch size has no instantiation (1, 2, 3, 5, 8, 32, 50)");                            \
    }

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
    if (src == nullptr || out == nullptr || rects == nullptr || dst_w <= 0 || dst_h <= 0) return bad_argument("null pointer or empty destination");
    if (!rects_inside(rects, n, src_w, src_h)) return bad_argument("crop rectangle outside the source image");
    return guarded([&]() -> int {
        Stream s(stream);
        int rc = FK_OK;
        FK_FOR_BATCH(n, (rc = readme_pipeline_any_ar<N>(s, aspect, src, src_w, src_h, src_pitch, rects, dst_w, dst_h, background, mul, sub, div, out)))
        return rc;
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
    if (srcs == nullptr || out == nullptr || rects == nullptr || dst_w <= 0 || dst_h <= 0) return bad_argument("null pointer or empty destination");
    if (!rects_inside(rects, n, src_w, src_h)) return bad_argument("crop rectangle outside the source image");
    return guarded([&]() -> int {
        Stream s(stream);
        FK_FOR_BATCH(n, (split_pipeline<N>(s, srcs, src_w, src_h, src_pitch, rects, dst_w, dst_h, div1, sub, div2, out)))
        return FK_OK;
    });
}

int fk_resize_crop_tiles(const void* src, int src_w, int src_h, size_t src_pitch, int rs_w, int rs_h, const fk_rect* rects, int n,
                         int tile_w, int tile_h, const float mul[3], float* out, void* stream) {
    if (src == nullptr || out == nullptr || rects == nullptr || rs_w <= 0 || rs_h <= 0) return bad_argument("null pointer or empty destination");
    if (!rects_inside(rects, n, rs_w, rs_h)) return bad_argument("tile outside the resized image");
    for (int i = 0; i < n; ++i) {
        if (rects[i].width != tile_w || rects[i].height != tile_h) return bad_argument("every tile must be tile_w x tile_h");
    }
    return guarded([&]() -> int {
        Stream s(stream);
        FK_FOR_BATCH(n, (tiles_pipeline<N>(s, src, src_w, src_h, src_pitch, rs_w, rs_h, rects, tile_w, tile_h, mul, out)))
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
    if (src == nullptr || out == nullptr || rects == nullptr) return bad_argument("null pointer");
    if (!rects_inside(rects, n, src_w, src_h)) return bad_argument("crop rectangle outside the source image");
    for (int i = 0; i < n; ++i) {
        if (rects[i].width > max_w || rects[i].height > max_h) return bad_argument("crop larger than the tensor plane");
    }
    return guarded([&]() -> int {
        Stream s(stream);
        FK_FOR_BATCH(n, (crops_pipeline<N>(s, src, src_w, src_h, src_pitch, rects, max_w, max_h, out)))
        return FK_OK;
    });
}

} // extern "C"
