// ref_driver_paths.cpp — drives the REFERENCE's own headers (its CPU backend, built exactly as they lie under
// /root/reference, nothing copied, no stand-in headers) behind the C signatures of fk_oracle_paths.h.
//
// TEST INFRASTRUCTURE ONLY.  Built by oracle/Makefile into oracle/_ref/libfkref_paths.so.  The reference fixes batch
// sizes at compile time: batches of 2, 3, 4 and 8 planes are instantiated here.
#include <fused_kernel/core/execution_model/memory_operations.h>
#include <fused_kernel/algorithms/basic_ops/arithmetic.h>
#include <fused_kernel/algorithms/basic_ops/cast.h>
#include <fused_kernel/algorithms/image_processing/crop.h>
#include <fused_kernel/algorithms/image_processing/resize.h>
#include <fused_kernel/algorithms/image_processing/saturate.h>
#include <fused_kernel/fused_kernel.h>

#include <array>
#include <cstddef>
#include <cstdint>

#include "fk_oracle_paths.h"

using namespace fk;

namespace {
using CPU = TransformDPP<ParArch::CPU>;

template <typename T>
RawPtr<ND::_2D, T> raw2d(const void* data, int w, int h, size_t pitch) {
    return RawPtr<ND::_2D, T>{ const_cast<T*>(static_cast<const T*>(data)),
                               PtrDims<ND::_2D>(static_cast<uint>(w), static_cast<uint>(h), static_cast<uint>(pitch)) };
}
template <typename T>
RawPtr<ND::_3D, T> raw3d(const void* data, int w, int h, int planes) {
    return RawPtr<ND::_3D, T>{ const_cast<T*>(static_cast<const T*>(data)),
                               PtrDims<ND::_3D>(static_cast<uint>(w), static_cast<uint>(h), static_cast<uint>(planes), 1u, static_cast<uint>(sizeof(T) * w)) };
}

template <size_t N>
void conditional_copy(const uint8_t* const* srcs, int w, int h, size_t pitch, int used, const uint8_t* def, uint8_t* out) {
    Stream_<ParArch::CPU> stream;
    std::array<RawPtr<ND::_2D, uchar3>, N> imgs;
    for (size_t i = 0; i < N; ++i) imgs[i] = raw2d<uchar3>(srcs[i], w, h, pitch);
    const auto read = PerThreadRead<ND::_2D, uchar3>::build(used, uchar3{ def[0], def[1], def[2] }, imgs);
    executeOperations<CPU>(stream, read, PerThreadWrite<ND::_3D, uchar3>::build(raw3d<uchar3>(out, w, h, static_cast<int>(N))));
}
template <size_t N>
void conditional_resize(const uint8_t* const* srcs, int w, int h, size_t pitch, int used, const float* def, int dw, int dh, float* out) {
    Stream_<ParArch::CPU> stream;
    std::array<RawPtr<ND::_2D, uchar3>, N> imgs;
    std::array<Size, N> sizes;
    for (size_t i = 0; i < N; ++i) {
        imgs[i] = raw2d<uchar3>(srcs[i], w, h, pitch);
        sizes[i] = Size(dw, dh);
    }
    const auto read = PerThreadRead<ND::_2D, uchar3>::build(imgs).then(
        Resize<InterpolationType::INTER_LINEAR>::build(used, float3{ def[0], def[1], def[2] }, sizes));
    executeOperations<CPU>(stream, read, TensorWrite<float3>::build(raw3d<float3>(out, dw, dh, static_cast<int>(N))));
}
template <size_t N>
void crop_cast_images(const uint8_t* src, int w, int h, size_t pitch, const fko_rect* rects, float* const* outs, size_t out_pitch) {
    Stream_<ParArch::CPU> stream;
    std::array<Rect, N> crops;
    std::array<RawPtr<ND::_2D, float3>, N> images;
    for (size_t i = 0; i < N; ++i) {
        crops[i] = Rect(static_cast<uint>(rects[i].x), static_cast<uint>(rects[i].y), rects[i].width, rects[i].height);
        images[i] = raw2d<float3>(outs[i], rects[i].width, rects[i].height, out_pitch);
    }
    const auto sender = PerThreadRead<ND::_2D, uchar3>::build(raw2d<uchar3>(src, w, h, pitch)).then(Crop<>::build(crops)).then(Cast<uchar3, float3>::build());
    executeOperations<CPU>(stream, sender, PerThreadWrite<ND::_2D, float3>::build(images));
}
// benchmark_horizontal_fusion.h:55-72: the batch is an array of windows of one image (Ptr2D::crop there, the same pointer
// arithmetic here), executeOperations(array, stream, ops..., TensorWrite)
template <size_t N>
void windows_saturate_muls(const uint8_t* src, int w, int h, size_t pitch, const fko_rect* rects, float mul_v, float sub_v, float div_v, float* out) {
    (void)w;
    (void)h;
    Stream_<ParArch::CPU> stream;
    std::array<RawPtr<ND::_2D, uchar>, N> crops;
    for (size_t i = 0; i < N; ++i) crops[i] = raw2d<uchar>(src + static_cast<size_t>(rects[i].y) * pitch + rects[i].x, rects[i].width, rects[i].height, pitch);
    const auto read = PerThreadRead<ND::_2D, uchar>::build(crops);
    executeOperations<CPU>(stream, read, SaturateCast<uchar, float>::build(), Mul<float>::build(mul_v), Sub<float>::build(sub_v), Div<float>::build(div_v),
                           TensorWrite<float>::build(raw3d<float>(out, rects[0].width, rects[0].height, static_cast<int>(N))));
}
} // namespace

#define FOR_BATCH(n, CALL)                                  \
    switch (n) {                                            \
    case 2: { constexpr size_t N = 2; CALL; return 0; }     \
    case 3: { constexpr size_t N = 3; CALL; return 0; }     \
    case 4: { constexpr size_t N = 4; CALL; return 0; }     \
    case 8: { constexpr size_t N = 8; CALL; return 0; }     \
    default: return 1;                                      \
    }

extern "C" {

int fkr_conditional_copy_u8c3(const uint8_t* const* srcs, int w, int h, size_t pitch, int n, int used, const uint8_t def[3], uint8_t* out) {
    FOR_BATCH(n, (conditional_copy<N>(srcs, w, h, pitch, used, def, out)))
}
int fkr_conditional_resize_f32c3(const uint8_t* const* srcs, int w, int h, size_t pitch, int n, int used, const float def[3], int dst_w,
                                 int dst_h, float* out) {
    FOR_BATCH(n, (conditional_resize<N>(srcs, w, h, pitch, used, def, dst_w, dst_h, out)))
}
int fkr_muladd_midwrite_f32c3(const float* src, int w, int h, size_t src_pitch, float mul_v, float add_v, float* mid, size_t mid_pitch,
                              float* out, size_t out_pitch) {
    Stream_<ParArch::CPU> stream;
    // the chain is fused with .then(): passed as separate arguments of executeOperations, the reference ends a chain at
    // its first write (data_parallel_patterns.h:77-79)
    const auto sender = PerThreadRead<ND::_2D, float3>::build(raw2d<float3>(src, w, h, src_pitch))
                            .then(Mul<float3>::build(make_set<float3>(mul_v)))
                            .then(PerThreadWrite<ND::_2D, float3>::build(raw2d<float3>(mid, w, h, mid_pitch)))
                            .then(Add<float3>::build(make_set<float3>(add_v)));
    executeOperations<CPU>(stream, sender, PerThreadWrite<ND::_2D, float3>::build(raw2d<float3>(out, w, h, out_pitch)));
    return 0;
}
int fkr_batch_crop_cast_images(const uint8_t* src, int w, int h, size_t pitch, const fko_rect* rects, int n, float* const* outs, size_t out_pitch) {
    FOR_BATCH(n, (crop_cast_images<N>(src, w, h, pitch, rects, outs, out_pitch)))
}
int fkr_batch_windows_saturate_muls_f32(const uint8_t* src, int w, int h, size_t pitch, const fko_rect* rects, int n, float mul_v, float sub_v,
                                        float div_v, float* out) {
    FOR_BATCH(n, (windows_saturate_muls<N>(src, w, h, pitch, rects, mul_v, sub_v, div_v, out)))
}
int fkr_tensor_mul_f32c3(const float* src, int w, int h, int planes, const float mul[3], float* out) {
    Stream_<ParArch::CPU> stream;
    executeOperations<CPU>(stream, TensorRead<float3>::build(raw3d<float3>(src, w, h, planes)), Mul<float3>::build(float3{ mul[0], mul[1], mul[2] }),
                           TensorWrite<float3>::build(raw3d<float3>(out, w, h, planes)));
    return 0;
}

} // extern "C"
