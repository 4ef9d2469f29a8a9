// ref_driver.cpp — drives the REFERENCE's own headers (its CPU backend, built exactly as they lie under
// /root/reference, nothing copied, no stand-in headers) behind the same C signatures as fk_oracle.h.
//
// TEST INFRASTRUCTURE ONLY.  Built by oracle/Makefile into oracle/_ref/libfkref.so when the reference tree is
// present; used to validate the C restatement in fk_oracle.c and as the "reference" CPU baseline.
//
// The host build of the reference takes the host branch of Interpolate (row index from the x coordinate,
// algorithms/image_processing/interpolation.h:69-70), so every resize chain here has the semantics that
// fk_oracle.c reproduces with quirk_y1_from_x = 1.  Callers keep inputs where that branch stays in bounds.
#include <fused_kernel/core/execution_model/memory_operations.h>
#include <fused_kernel/core/utils/utils.h>
#include <fused_kernel/algorithms/basic_ops/arithmetic.h>
#include <fused_kernel/algorithms/basic_ops/cast.h>
#include <fused_kernel/algorithms/image_processing/crop.h>
#include <fused_kernel/algorithms/image_processing/color_conversion.h>
#include <fused_kernel/algorithms/image_processing/resize.h>
#include <fused_kernel/algorithms/image_processing/saturate.h>
#include <fused_kernel/fused_kernel.h>

#include <array>
#include <cstdint>
#include <cstddef>

#include "fk_oracle.h"

using namespace fk;

namespace {
using CPU = TransformDPP<ParArch::CPU>;

template <typename T>
RawPtr<ND::_2D, T> raw2d(const void* data, int w, int h, size_t pitch) {
    return RawPtr<ND::_2D, T>{ const_cast<T*>(static_cast<const T*>(data)),
                               PtrDims<ND::_2D>(static_cast<uint>(w), static_cast<uint>(h), static_cast<uint>(pitch)) };
}
template <typename T>
RawPtr<ND::_3D, T> raw3d(void* data, int w, int h, int planes, int color_planes) {
    return RawPtr<ND::_3D, T>{ static_cast<T*>(data),
                               PtrDims<ND::_3D>(static_cast<uint>(w), static_cast<uint>(h), static_cast<uint>(planes),
                                                static_cast<uint>(color_planes), static_cast<uint>(sizeof(T) * w)) };
}
template <size_t N>
std::array<Rect, N> rect_array(const fko_rect* r) {
    std::array<Rect, N> a;
    for (size_t i = 0; i < N; ++i) a[i] = Rect(static_cast<uint>(r[i].x), static_cast<uint>(r[i].y), r[i].width, r[i].height);
    return a;
}
float3 f3(const float* v) { return float3{ v[0], v[1], v[2] }; }

template <size_t N, AspectRatio AR>
void readme_chain(const uint8_t* src, int w, int h, size_t pitch, const fko_rect* rects, int dw, int dh,
                  const float* bg, const float* mul, const float* sub, const float* div, float* out) {
    Stream_<ParArch::CPU> stream;
    const auto crops = rect_array<N>(rects);
    const auto read = PerThreadRead<ND::_2D, uchar3>::build(raw2d<uchar3>(src, w, h, pitch)).then(Crop<>::build(crops));
    const auto write = TensorWrite<float3>::build(raw3d<float3>(out, dw, dh, static_cast<int>(N), 1));
    if constexpr (AR == AspectRatio::IGNORE_AR) {
        const auto sender = read.then(Resize<InterpolationType::INTER_LINEAR, AR>::build(Size(dw, dh)))
                                .then(Mul<float3>::build(f3(mul)))
                                .then(Sub<float3>::build(f3(sub)))
                                .then(Div<float3>::build(f3(div)))
                                .then(ColorConversion<ColorConversionCodes::COLOR_RGB2BGR, float3, float3>::build());
        executeOperations<CPU>(stream, sender, write);
    } else {
        const auto sender = read.then(Resize<InterpolationType::INTER_LINEAR, AR>::build(Size(dw, dh), f3(bg)))
                                .then(Mul<float3>::build(f3(mul)))
                                .then(Sub<float3>::build(f3(sub)))
                                .then(Div<float3>::build(f3(div)))
                                .then(ColorConversion<ColorConversionCodes::COLOR_RGB2BGR, float3, float3>::build());
        executeOperations<CPU>(stream, sender, write);
    }
}

template <size_t N>
void readme_chain_ar(const uint8_t* src, int w, int h, size_t pitch, const fko_rect* rects, int dw, int dh, int aspect,
                     const float* bg, const float* mul, const float* sub, const float* div, float* out) {
    switch (aspect) {
    case FKO_PRESERVE_AR: readme_chain<N, AspectRatio::PRESERVE_AR>(src, w, h, pitch, rects, dw, dh, bg, mul, sub, div, out); break;
    case FKO_IGNORE_AR: readme_chain<N, AspectRatio::IGNORE_AR>(src, w, h, pitch, rects, dw, dh, bg, mul, sub, div, out); break;
    case FKO_PRESERVE_AR_RN_EVEN: readme_chain<N, AspectRatio::PRESERVE_AR_RN_EVEN>(src, w, h, pitch, rects, dw, dh, bg, mul, sub, div, out); break;
    default: readme_chain<N, AspectRatio::PRESERVE_AR_LEFT>(src, w, h, pitch, rects, dw, dh, bg, mul, sub, div, out); break;
    }
}

template <size_t N>
void split_chain(const uint8_t* const* srcs, int w, int h, size_t pitch, const fko_rect* rects, int dw, int dh,
                 const float* d1, const float* s, const float* d2, float* out) {
    Stream_<ParArch::CPU> stream;
    std::array<RawPtr<ND::_2D, uchar3>, N> imgs;
    for (size_t i = 0; i < N; ++i) imgs[i] = raw2d<uchar3>(srcs[i], w, h, pitch);
    const auto sender = PerThreadRead<ND::_2D, uchar3>::build(imgs)
                            .then(Crop<>::build(rect_array<N>(rects)))
                            .then(Resize<InterpolationType::INTER_LINEAR>::build(Size(dw, dh)))
                            .then(Div<float3>::build(f3(d1)))
                            .then(Sub<float3>::build(f3(s)))
                            .then(Div<float3>::build(f3(d2)))
                            .then(ColorConversion<ColorConversionCodes::COLOR_RGB2BGR, float3, float3>::build());
    const auto write = TensorSplit<float3>::build(raw3d<float>(out, dw, dh, static_cast<int>(N), 3));
    executeOperations<CPU>(stream, sender, write);
}

template <size_t N>
void tiles_chain(const uint8_t* src, int w, int h, size_t pitch, int rw, int rh, const fko_rect* rects, int tw, int th,
                 const float* mul, float* out) {
    Stream_<ParArch::CPU> stream;
    const auto sender = PerThreadRead<ND::_2D, uchar3>::build(raw2d<uchar3>(src, w, h, pitch))
                            .then(Resize<InterpolationType::INTER_LINEAR>::build(Size(rw, rh)))
                            .then(Crop<>::build(rect_array<N>(rects)))
                            .then(Mul<float3>::build(f3(mul)));
    const auto write = TensorWrite<float3>::build(raw3d<float3>(out, tw, th, static_cast<int>(N), 1));
    executeOperations<CPU>(stream, sender, write);
}

template <size_t N>
void crops_chain(const uint8_t* src, int w, int h, size_t pitch, const fko_rect* rects, int mw, int mh, float* out) {
    Stream_<ParArch::CPU> stream;
    const auto sender = PerThreadRead<ND::_2D, uchar3>::build(raw2d<uchar3>(src, w, h, pitch))
                            .then(Crop<>::build(rect_array<N>(rects)))
                            .then(Cast<uchar3, float3>::build());
    const auto write = TensorWrite<float3>::build(raw3d<float3>(out, mw, mh, static_cast<int>(N), 1));
    executeOperations<CPU>(stream, sender, write);
}

template <int DEPTH, int K = 0, typename Sender>
void muladd_rec(Stream_<ParArch::CPU>& stream, const Sender& sender, float mul_v, float add_v,
                const Write<PerThreadWrite<ND::_2D, float3>>& write) {
    if constexpr (K == DEPTH) {
        executeOperations<CPU>(stream, sender, write);
    } else if constexpr (K % 2 == 1) {
        muladd_rec<DEPTH, K + 1>(stream, sender.then(Add<float3>::build(make_set<float3>(add_v))), mul_v, add_v, write);
    } else {
        muladd_rec<DEPTH, K + 1>(stream, sender.then(Mul<float3>::build(make_set<float3>(mul_v))), mul_v, add_v, write);
    }
}
} // namespace

#define FKR_BATCH_SWITCH(n, CALL)                                                                                       \
    switch (n) {                                                                                                       \
    case 1: { constexpr size_t N = 1; CALL; return 0; }                                                                \
    case 2: { constexpr size_t N = 2; CALL; return 0; }                                                                \
    case 3: { constexpr size_t N = 3; CALL; return 0; }                                                                \
    case 5: { constexpr size_t N = 5; CALL; return 0; }                                                                \
    case 8: { constexpr size_t N = 8; CALL; return 0; }                                                                \
    case 32: { constexpr size_t N = 32; CALL; return 0; }                                                              \
    case 50: { constexpr size_t N = 50; CALL; return 0; }                                                              \
    default: return 1;                                                                                                 \
    }

extern "C" {

// returns 0, or 1 when the batch size is not one the driver was instantiated for
int fkr_crop_resize_muls_bgr_tensor(const uint8_t* src, int src_w, int src_h, size_t src_pitch, const fko_rect* rects,
                                    int n, int dst_w, int dst_h, int aspect, const float* background,
                                    const float* mul, const float* sub, const float* div, float* out) {
    FKR_BATCH_SWITCH(n, (readme_chain_ar<N>(src, src_w, src_h, src_pitch, rects, dst_w, dst_h, aspect, background, mul, sub, div, out)))
}

int fkr_batch_crop_resize_norm_split(const uint8_t* const* srcs, int src_w, int src_h, size_t src_pitch,
                                     const fko_rect* rects, int n, int dst_w, int dst_h, const float* div1,
                                     const float* sub, const float* div2, float* out) {
    FKR_BATCH_SWITCH(n, (split_chain<N>(srcs, src_w, src_h, src_pitch, rects, dst_w, dst_h, div1, sub, div2, out)))
}

int fkr_resize_crop_tiles(const uint8_t* src, int src_w, int src_h, size_t src_pitch, int rs_w, int rs_h,
                          const fko_rect* rects, int n, int tile_w, int tile_h, const float* mul, float* out) {
    FKR_BATCH_SWITCH(n, (tiles_chain<N>(src, src_w, src_h, src_pitch, rs_w, rs_h, rects, tile_w, tile_h, mul, out)))
}

int fkr_batch_crop_cast_tensor(const uint8_t* src, int src_w, int src_h, size_t src_pitch, const fko_rect* rects, int n,
                               int max_w, int max_h, float* out) {
    FKR_BATCH_SWITCH(n, (crops_chain<N>(src, src_w, src_h, src_pitch, rects, max_w, max_h, out)))
}

int fkr_muladd_chain_f32c3(const float* src, int w, int h, size_t src_pitch, int depth, float mul_v, float add_v,
                           float* dst, size_t dst_pitch) {
    Stream_<ParArch::CPU> stream;
    const auto read = PerThreadRead<ND::_2D, float3>::build(raw2d<float3>(src, w, h, src_pitch));
    const auto write = PerThreadWrite<ND::_2D, float3>::build(raw2d<float3>(dst, w, h, dst_pitch));
    switch (depth) {
    case 1: muladd_rec<1>(stream, read, mul_v, add_v, write); return 0;
    case 2: muladd_rec<2>(stream, read, mul_v, add_v, write); return 0;
    case 4: muladd_rec<4>(stream, read, mul_v, add_v, write); return 0;
    case 8: muladd_rec<8>(stream, read, mul_v, add_v, write); return 0;
    case 16: muladd_rec<16>(stream, read, mul_v, add_v, write); return 0;
    default: return 1;
    }
}

int fkr_single_op_f32c3(const float* src, int w, int h, size_t src_pitch, int is_add, float v, float* dst,
                        size_t dst_pitch) {
    Stream_<ParArch::CPU> stream;
    const auto read = PerThreadRead<ND::_2D, float3>::build(raw2d<float3>(src, w, h, src_pitch));
    const auto write = PerThreadWrite<ND::_2D, float3>::build(raw2d<float3>(dst, w, h, dst_pitch));
    if (is_add) executeOperations<CPU>(stream, read, Add<float3>::build(make_set<float3>(v)), write);
    else executeOperations<CPU>(stream, read, Mul<float3>::build(make_set<float3>(v)), write);
    return 0;
}

int fkr_rgba2gray_u8c4(const uint8_t* src, int w, int h, size_t src_pitch, uint8_t* dst, size_t dst_pitch) {
    Stream_<ParArch::CPU> stream;
    executeOperations<CPU>(stream, PerThreadRead<ND::_2D, uchar4>::build(raw2d<uchar4>(src, w, h, src_pitch)),
                           ColorConversion<ColorConversionCodes::COLOR_RGBA2GRAY, uchar4, uchar>::build(),
                           PerThreadWrite<ND::_2D, uchar>::build(raw2d<uchar>(dst, w, h, dst_pitch)));
    return 0;
}

int fkr_resize_mul_u8c4_f32c4(const uint8_t* src, int w, int h, size_t src_pitch, int dst_w, int dst_h, float mul_v,
                              float* dst, size_t dst_pitch) {
    Stream_<ParArch::CPU> stream;
    const auto sender = PerThreadRead<ND::_2D, uchar4>::build(raw2d<uchar4>(src, w, h, src_pitch))
                            .then(Resize<InterpolationType::INTER_LINEAR>::build(Size(dst_w, dst_h)))
                            .then(Mul<float4>::build(make_set<float4>(mul_v)));
    executeOperations<CPU>(stream, sender, PerThreadWrite<ND::_2D, float4>::build(raw2d<float4>(dst, dst_w, dst_h, dst_pitch)));
    return 0;
}

int fkr_crop_mul_saturate_u8c4(const uint8_t* src, int w, int h, size_t src_pitch, fko_rect rect, int mul_v,
                               uint8_t* dst, size_t dst_pitch) {
    Stream_<ParArch::CPU> stream;
    const auto sender = PerThreadRead<ND::_2D, uchar4>::build(raw2d<uchar4>(src, w, h, src_pitch))
                            .then(Crop<>::build(Rect(static_cast<uint>(rect.x), static_cast<uint>(rect.y), rect.width, rect.height)))
                            .then(Mul<uchar4, int, int4>::build(mul_v))
                            .then(SaturateCast<int4, uchar4>::build());
    executeOperations<CPU>(stream, sender,
                           PerThreadWrite<ND::_2D, uchar4>::build(raw2d<uchar4>(dst, rect.width, rect.height, dst_pitch)));
    return 0;
}

int fkr_rgba2bgr_sub_u8c4_f32c3(const uint8_t* src, int w, int h, size_t src_pitch, float sub_v, float* dst,
                                size_t dst_pitch) {
    Stream_<ParArch::CPU> stream;
    executeOperations<CPU>(stream, PerThreadRead<ND::_2D, uchar4>::build(raw2d<uchar4>(src, w, h, src_pitch)),
                           ColorConversion<ColorConversionCodes::COLOR_RGBA2BGR, uchar4, uchar3>::build(),
                           Cast<uchar3, float3>::build(), Sub<float3>::build(make_set<float3>(sub_v)),
                           PerThreadWrite<ND::_2D, float3>::build(raw2d<float3>(dst, w, h, dst_pitch)));
    return 0;
}

// Known-answer probes of single reference operations, for the oracle's building blocks.
float fkr_cxp_round(float x) { return cxp::round(x); }
uint8_t fkr_saturate_float_to_u8(float v) { return SaturateCast<float, uchar>::exec(v); }
uint8_t fkr_saturate_int_to_u8(int v) { return SaturateCast<int, uchar>::exec(v); }
uint8_t fkr_rgb2gray_u8(uint8_t x, uint8_t y, uint8_t z) {
    return ColorConversion<ColorConversionCodes::COLOR_RGB2GRAY, uchar3, uchar>::exec(uchar3{ x, y, z });
}

} // extern "C"
