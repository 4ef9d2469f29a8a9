// fk_capi_paths.hip — entry points of include/fk_capi.h for the operator API's less common chain shapes: batch reads with
// PlanePolicy::CONDITIONAL_WITH_DEFAULT, a write in the middle of a chain, a batch of separate output images and a
// tensor as the source.  Compiled by hipcc into libfk_capi.so.
#include <array>

#include "fk_capi_common.h"

using namespace fk;
using namespace fk_capi;

namespace {
constexpr int MAX_PLANES = 64;

// The operator API fixes a batch's size at compile time; a batch of n planes is built with a capacity of 8 or 64, its
// unused entries repeat the first, and its thread grid is cut to n planes.
template <size_t CAP, typename T>
std::array<RawPtr<ND::_2D, T>, CAP> images_of(const void* const* ptrs, int n, int w, int h, size_t pitch) {
    std::array<RawPtr<ND::_2D, T>, CAP> images;
    for (size_t i = 0; i < CAP; ++i) images[i] = view2d<T>(ptrs[i < static_cast<size_t>(n) ? i : 0], w, h, pitch);
    return images;
}
template <typename BatchIOp>
BatchIOp with_planes(BatchIOp batch, int n) {
    batch.params.activeThreads.z = static_cast<uint>(n);
    return batch;
}

template <size_t CAP>
void conditional_copy(Stream& stream, const void* const* srcs, int w, int h, size_t pitch, int n, int used, const uint8_t* def, void* out) {
    const auto read = PerThreadRead<ND::_2D, uchar3>::build(used, uchar3{ def[0], def[1], def[2] }, images_of<CAP, uchar3>(srcs, n, w, h, pitch));
    executeOperations<TransformDPP<>>(stream, with_planes(read, n), PerThreadWrite<ND::_3D, uchar3>::build(view3d<uchar3>(out, w, h, n, 1)));
}
template <size_t CAP>
void conditional_resize(Stream& stream, const void* const* srcs, int w, int h, size_t pitch, int n, int used, const float* def, int dw, int dh,
                        float* out) {
    std::array<Size, CAP> sizes;
    sizes.fill(Size(dw, dh));
    const auto read = PerThreadRead<ND::_2D, uchar3>::build(images_of<CAP, uchar3>(srcs, n, w, h, pitch))
                          .then(Resize<InterpolationType::INTER_LINEAR>::build(used, float3{ def[0], def[1], def[2] }, sizes));
    executeOperations<TransformDPP<>>(stream, with_planes(read, n), TensorWrite<float3>::build(view3d<float3>(out, dw, dh, n, 1)));
}
template <size_t CAP>
void crop_cast_images(Stream& stream, const void* src, int w, int h, size_t pitch, const fk_rect* rects, int n, float* const* outs, size_t out_pitch) {
    std::array<Rect, CAP> crops;
    std::array<RawPtr<ND::_2D, float3>, CAP> images;
    for (size_t i = 0; i < CAP; ++i) {
        const size_t k = i < static_cast<size_t>(n) ? i : 0;
        crops[i] = Rect(static_cast<uint>(rects[k].x), static_cast<uint>(rects[k].y), rects[k].width, rects[k].height);
        images[i] = view2d<float3>(outs[k], rects[k].width, rects[k].height, out_pitch);
    }
    const auto sender = PerThreadRead<ND::_2D, uchar3>::build(view2d<uchar3>(src, w, h, pitch)).then(Crop<>::build(crops)).then(Cast<uchar3, float3>::build());
    executeOperations<TransformDPP<>>(stream, with_planes(sender, n), PerThreadWrite<ND::_2D, float3>::build(images));
}
} // namespace

#define FK_FOR_CAPACITY(n, CALL)                         \
    if ((n) <= 8) { constexpr size_t CAP = 8; CALL; }    \
    else { constexpr size_t CAP = MAX_PLANES; CALL; }

extern "C" {

int fk_conditional_copy_u8c3(const void* const* srcs, int w, int h, size_t pitch, int n, int used, const uint8_t def[3], void* out, void* stream) {
    if (srcs == nullptr || out == nullptr || def == nullptr || w <= 0 || h <= 0) return bad_argument("null pointer or empty image");
    if (n <= 0 || n > MAX_PLANES) return bad_argument("a conditional batch takes 1 to 64 planes");
    return guarded([&]() -> int {
        Stream s(stream);
        FK_FOR_CAPACITY(n, (conditional_copy<CAP>(s, srcs, w, h, pitch, n, used, def, out)))
        return FK_OK;
    });
}

int fk_conditional_resize_f32c3(const void* const* srcs, int w, int h, size_t pitch, int n, int used, const float def[3], int dst_w, int dst_h,
                                float* out, void* stream) {
    if (srcs == nullptr || out == nullptr || def == nullptr || w <= 0 || h <= 0 || dst_w <= 0 || dst_h <= 0) return bad_argument("null pointer or empty image");
    if (n <= 0 || n > MAX_PLANES) return bad_argument("a conditional batch takes 1 to 64 planes");
    if (!interpolation_rows_exist(0, w, h)) return rows_missing();
    return guarded([&]() -> int {
        Stream s(stream);
        FK_FOR_CAPACITY(n, (conditional_resize<CAP>(s, srcs, w, h, pitch, n, used, def, dst_w, dst_h, out)))
        return FK_OK;
    });
}

int fk_muladd_midwrite_f32c3(const void* src, int w, int h, size_t src_pitch, float mul_v, float add_v, void* mid, size_t mid_pitch, void* out,
                             size_t out_pitch, void* stream) {
    if (src == nullptr || mid == nullptr || out == nullptr || w <= 0 || h <= 0) return bad_argument("null pointer or empty image");
    return guarded([&]() -> int {
        Stream s(stream);
        executeOperations<TransformDPP<>>(s, PerThreadRead<ND::_2D, float3>::build(view2d<float3>(src, w, h, src_pitch)),
                                          Mul<float3>::build(make_set<float3>(mul_v)), PerThreadWrite<ND::_2D, float3>::build(view2d<float3>(mid, w, h, mid_pitch)),
                                          Add<float3>::build(make_set<float3>(add_v)), PerThreadWrite<ND::_2D, float3>::build(view2d<float3>(out, w, h, out_pitch)));
        return FK_OK;
    });
}

int fk_batch_crop_cast_images(const void* src, int w, int h, size_t pitch, const fk_rect* rects, int n, float* const* outs, size_t out_pitch,
                              void* stream) {
    if (src == nullptr || rects == nullptr || outs == nullptr) return bad_argument("null pointer");
    if (n <= 0 || n > MAX_PLANES) return bad_argument("a batch of output images takes 1 to 64 planes");
    for (int i = 0; i < n; ++i) {
        const fk_rect& r = rects[i];
        if (outs[i] == nullptr) return bad_argument("null pointer");
        if (r.x < 0 || r.y < 0 || r.width <= 0 || r.height <= 0 || r.x + r.width > w || r.y + r.height > h) return bad_argument("crop rectangle outside the source image");
        if (r.width != rects[0].width || r.height != rects[0].height) return bad_argument("every crop must have the size of the first");
    }
    return guarded([&]() -> int {
        Stream s(stream);
        FK_FOR_CAPACITY(n, (crop_cast_images<CAP>(s, src, w, h, pitch, rects, n, outs, out_pitch)))
        return FK_OK;
    });
}

int fk_tensor_mul_f32c3(const void* src, int w, int h, int planes, const float mul[3], void* out, void* stream) {
    if (src == nullptr || out == nullptr || mul == nullptr || w <= 0 || h <= 0 || planes <= 0) return bad_argument("null pointer or empty tensor");
    return guarded([&]() -> int {
        Stream s(stream);
        executeOperations<TransformDPP<>>(s, TensorRead<float3>::build(view3d<float3>(const_cast<void*>(src), w, h, planes, 1)),
                                          Mul<float3>::build(float3{ mul[0], mul[1], mul[2] }), TensorWrite<float3>::build(view3d<float3>(out, w, h, planes, 1)));
        return FK_OK;
    });
}

int fk_set_to_f32c3_tensor(const float value[3], void* out, int w, int h, int planes, void* stream) {
    if (out == nullptr || value == nullptr || w <= 0 || h <= 0 || planes <= 0) return bad_argument("null pointer or empty tensor");
    return guarded([&]() -> int {
        Stream s(stream);
        // what fk::setTo launches for a Tensor<float3> in device memory
        const ActiveThreads extent(static_cast<uint>(w), static_cast<uint>(h), static_cast<uint>(planes));
        executeOperations<TransformDPP<>>(s, ReadSet<float3>::build(float3{ value[0], value[1], value[2] }, extent),
                                          PerThreadWrite<ND::_3D, float3>::build(view3d<float3>(out, w, h, planes, 1)));
        return FK_OK;
    });
}

} // extern "C"
