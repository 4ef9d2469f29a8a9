// YUV front-end of the fused Transform path: raw YUV images, ReadYUV / WriteYUV and ConvertYUVToRGB.
//
// Same names, template parameters and arithmetic as the reference's algorithms/image_processing/raw_image.h:23-114
// (ColorSpace, ColorRange, ColorPrimitives, PixelFormat, PixelFormatTraits, RawImage), image.h:22-92 (Image),
// color_conversion.h:87-103,132-195 (constants), :197-310 (pixel normalisation, ConvertYUVToRGB), :315-400 (ReadYUV),
// :402-513 (WriteYUV), basic_ops/algebraic.h:24-48 (M3x3Float, MxVFloat3) and logical.h:23-82 (shifts, IsEven).
//
// Formats whose traits the reference defines and whose read compiles there are supported: NV12, NV21, P010, P210,
// Y210, UYVY.  One thing differs on purpose: the chroma plane of the semi-planar formats starts `pitch * image height`
// bytes after the luma plane.  The reference offsets it by `pitch * data.dims.height` (color_conversion.h:337,353),
// which is the same address only when the RawImage's data dims carry the image height; for an Image<PF> allocated by
// its own constructor (data height = 1.5 x image height) that offset lies past the allocation.
#ifndef FK_OPS_YUV_H
#define FK_OPS_YUV_H

#include "fk/ops/arithmetic.h"
#include "fk/ops/image_processing.h"
#include "fk/ops/memory_operations.h"

namespace fk {

enum class ColorSpace { YUV420, YUV422, YUV444, RGB, RGBA };
enum class ColorRange { Limited, Full };
enum class ColorPrimitives { bt601, bt709, bt2020 };
enum class PixelFormat { NV12, NV21, YV12, P010, P016, P216, P210, Y216, Y210, Y416, UYVY };

namespace detail {
template <ColorDepth CD> struct DepthBase { using type = ushort; };
template <> struct DepthBase<ColorDepth::p8bit> { using type = uchar; };
template <> struct DepthBase<ColorDepth::f24bit> { using type = float; };
} // namespace detail
template <ColorDepth CD>
using ColorDepthPixelBaseType = typename detail::DepthBase<CD>::type;
template <ColorDepth CD>
using ColorDepthPixelType = VectorType_t<ColorDepthPixelBaseType<CD>, 3>;

// Elements of the pixel base type per image pixel, along x and along y.
struct ResolutionFactors {
    float width_f;
    float height_f;
};

template <PixelFormat PF>
struct PixelFormatTraits;
#define FK_PIXEL_FORMAT(PF, SPACE, DEPTH, CN, RFW, RFH)                                                                \
    template <>                                                                                                        \
    struct PixelFormatTraits<PixelFormat::PF> {                                                                        \
        static constexpr ColorSpace space = ColorSpace::SPACE;                                                         \
        static constexpr ColorDepth depth = ColorDepth::DEPTH;                                                         \
        static constexpr size_t cn = CN;                                                                               \
        static constexpr ResolutionFactors rf{ RFW, RFH };                                                             \
    };
FK_PIXEL_FORMAT(NV12, YUV420, p8bit, 3, 1.f, 1.5f)
FK_PIXEL_FORMAT(NV21, YUV420, p8bit, 3, 1.f, 1.5f)
FK_PIXEL_FORMAT(YV12, YUV420, p8bit, 3, 1.f, 1.5f)
FK_PIXEL_FORMAT(P010, YUV420, p10bit, 3, 1.f, 1.5f)
FK_PIXEL_FORMAT(P210, YUV422, p10bit, 3, 1.f, 2.f)
FK_PIXEL_FORMAT(Y210, YUV422, p10bit, 3, 2.f, 1.f)
FK_PIXEL_FORMAT(Y416, YUV444, p12bit, 4, 4.f, 1.f)
FK_PIXEL_FORMAT(UYVY, YUV422, p8bit, 3, 2.f, 1.f)
#undef FK_PIXEL_FORMAT

// The buffer of a YUV image (all planes in one 2D allocation) plus the image size in pixels.
template <PixelFormat PF>
struct RawImage {
    using BaseType = ColorDepthPixelBaseType<PixelFormatTraits<PF>::depth>;
    RawPtr<ND::_2D, BaseType> data;
    uint width;
    uint height;
};

template <PixelFormat PF>
using PackedPixelType = VectorType_t<ColorDepthPixelBaseType<PixelFormatTraits<PF>::depth>, static_cast<int>(PixelFormatTraits<PF>::cn)>;
template <PixelFormat PF, bool ALPHA>
using YUVOutputPixelType =
    VectorType_t<ColorDepthPixelBaseType<PixelFormatTraits<PF>::depth>, ALPHA ? 4 : static_cast<int>(PixelFormatTraits<PF>::cn)>;

// ---- per-depth constants -------------------------------------------------------------------------------------
struct SubCoefficients {
    float luma;
    float chroma;
};
template <ColorDepth CD> constexpr SubCoefficients subCoefficients{};
template <> inline constexpr SubCoefficients subCoefficients<ColorDepth::p8bit>{ 16.f, 128.f };
template <> inline constexpr SubCoefficients subCoefficients<ColorDepth::p10bit>{ 64.f, 512.f };
template <> inline constexpr SubCoefficients subCoefficients<ColorDepth::p12bit>{ 64.f, 2048.f };

template <ColorDepth CD> constexpr ColorDepthPixelBaseType<CD> maxDepthValue{};
template <> inline constexpr uchar maxDepthValue<ColorDepth::p8bit>{ 255u };
template <> inline constexpr ushort maxDepthValue<ColorDepth::p10bit>{ 1023u };
template <> inline constexpr ushort maxDepthValue<ColorDepth::p12bit>{ 4095u };
template <> inline constexpr float maxDepthValue<ColorDepth::f24bit>{ 1.f };

// Samples of 10- and 12-bit formats sit in the high bits of a 16-bit word.
template <ColorDepth CD> constexpr ColorDepthPixelBaseType<CD> shiftFactor{};
template <> inline constexpr uchar shiftFactor<ColorDepth::p8bit>{ 0u };
template <> inline constexpr ushort shiftFactor<ColorDepth::p10bit>{ 6u };
template <> inline constexpr ushort shiftFactor<ColorDepth::p12bit>{ 4u };
template <ColorDepth CD> constexpr float floatShiftFactor{};
template <> inline constexpr float floatShiftFactor<ColorDepth::p8bit>{ 1.f };
template <> inline constexpr float floatShiftFactor<ColorDepth::p10bit>{ 64.f };
template <> inline constexpr float floatShiftFactor<ColorDepth::p12bit>{ 16.f };

// ---- 3x3 matrix times vector ---------------------------------------------------------------------------------
struct M3x3Float {
    float3 x;
    float3 y;
    float3 z;
};

// Row r of the result is (v.x*m.r.x + v.y*m.r.y) + v.z*m.r.z.
template <typename OpInstanceType = BinaryType>
struct MxVFloat3;
template <>
struct MxVFloat3<BinaryType> {
private:
    using SelfType = MxVFloat3<BinaryType>;
    FK_HD_STATIC float dot(const float3& v, const float3& row) { return (v.x * row.x + v.y * row.y) + v.z * row.z; }

public:
    FK_BINARY_OPERATION(MxVFloat3, float3, M3x3Float, float3)
    FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) {
        return float3{ dot(input, params.x), dot(input, params.y), dot(input, params.z) };
    }
};

enum class ColorConversionDir { YCbCr2RGB, RGB2YCbCr };

// Combinations without a specialisation are the zero matrix, as in the reference (color_conversion.h:134-135).
template <ColorRange CR, ColorPrimitives CP, ColorConversionDir CCD>
constexpr M3x3Float ccMatrix{};
template <>
inline constexpr M3x3Float ccMatrix<ColorRange::Full, ColorPrimitives::bt601, ColorConversionDir::YCbCr2RGB>{
    { 1.164383562f, 0.f, 1.596026786f }, { 1.164383562f, -0.39176229f, -0.812967647f }, { 1.164383562f, 2.017232143f, 0.f } };
template <>
inline constexpr M3x3Float ccMatrix<ColorRange::Full, ColorPrimitives::bt709, ColorConversionDir::YCbCr2RGB>{
    { 1.f, 0.f, 1.5748f }, { 1.f, -0.1873f, -0.4681f }, { 1.f, 1.8556f, 0.f } };
template <>
inline constexpr M3x3Float ccMatrix<ColorRange::Limited, ColorPrimitives::bt709, ColorConversionDir::YCbCr2RGB>{
    { 1.f, 0.f, 1.402f }, { 1.f, -0.34414f, -0.71414f }, { 1.f, 1.772f, 0.f } };
template <>
inline constexpr M3x3Float ccMatrix<ColorRange::Full, ColorPrimitives::bt709, ColorConversionDir::RGB2YCbCr>{
    { 0.2126f, 0.7152f, 0.0722f }, { -0.1146f, -0.3854f, 0.5f }, { 0.5f, -0.4542f, -0.0458f } };
template <>
inline constexpr M3x3Float ccMatrix<ColorRange::Full, ColorPrimitives::bt2020, ColorConversionDir::YCbCr2RGB>{
    { 1.f, 0.f, 1.4746f }, { 1.f, -0.16455312684366f, -0.57135312684366f }, { 1.f, 1.8814f, 0.f } };
template <>
inline constexpr M3x3Float ccMatrix<ColorRange::Full, ColorPrimitives::bt2020, ColorConversionDir::RGB2YCbCr>{
    { -0.73792134831461f, 1.90449438202248f, -0.16657303370787f },
    { 0.39221927730127f, -1.01227510472121f, 0.62005582741994f },
    { 1.17857137414527f, -1.29153287808387f, 0.11296150393861f } };

// ---- bit shifts and parity -----------------------------------------------------------------------------------
enum class ShiftDirection { Left, Right };
template <typename T, ShiftDirection SD>
struct Shift {
private:
    using SelfType = Shift<T, SD>;
    using B = VBase<T>;
    static_assert(std::is_unsigned_v<B>, "Shift only works with unsigned integers.");
    FK_HD_STATIC B one(const B v, const uint n) {
        if constexpr (SD == ShiftDirection::Left) return static_cast<B>(v << n);
        else return static_cast<B>(v >> n);
    }

public:
    FK_BINARY_OPERATION(Shift, T, uint, T)
    FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) {
        if constexpr (!validCUDAVec<T>) return one(input, params);
        else if constexpr (cn<T> == 1) return T{ one(input.x, params) };
        else if constexpr (cn<T> == 2) return T{ one(input.x, params), one(input.y, params) };
        else if constexpr (cn<T> == 3) return T{ one(input.x, params), one(input.y, params), one(input.z, params) };
        else return T{ one(input.x, params), one(input.y, params), one(input.z, params), one(input.w, params) };
    }
};
template <typename T> using ShiftLeft = Shift<T, ShiftDirection::Left>;
template <typename T> using ShiftRight = Shift<T, ShiftDirection::Right>;

template <typename I>
struct IsEven {
private:
    using SelfType = IsEven<I>;

public:
    FK_UNARY_OPERATION(IsEven, I, bool)
    static_assert(std::is_integral_v<I>, "Input type not valid for IsEven");
    FK_HD_STATIC OutputType exec(const InputType& input) { return (static_cast<std::make_unsigned_t<I>>(input) & 1u) == 0; }
};

// ---- normalised pixels ---------------------------------------------------------------------------------------
template <typename I, ColorDepth CD>
struct NormalizePixel {
private:
    using SelfType = NormalizePixel<I, CD>;
    using O_ = VectorType_t<float, cn<I>>;

public:
    FK_UNARY_OPERATION(NormalizePixel, I, O_)
    FK_HD_STATIC OutputType exec(const InputType& input) { return input / static_cast<float>(maxDepthValue<CD>); }
};
template <typename O, ColorDepth CD>
struct DenormalizePixel {
private:
    using SelfType = DenormalizePixel<O, CD>;
    using I_ = VectorType_t<float, cn<O>>;

public:
    FK_UNARY_OPERATION(DenormalizePixel, I_, O)
    FK_HD_STATIC OutputType exec(const InputType& input) {
        return Cast<InputType, OutputType>::exec(input * static_cast<float>(maxDepthValue<CD>));
    }
};
namespace detail {
FK_HD_CNST float clamp_float(const float v, const float lo, const float hi) { return cxp::max(lo, cxp::min(v, hi)); }
template <typename T>
FK_HD_CNST T clamp_channels(const T& v, const float lo, const float hi) {
    if constexpr (!validCUDAVec<T>) return clamp_float(v, lo, hi);
    else if constexpr (cn<T> == 1) return T{ clamp_float(v.x, lo, hi) };
    else if constexpr (cn<T> == 2) return T{ clamp_float(v.x, lo, hi), clamp_float(v.y, lo, hi) };
    else if constexpr (cn<T> == 3) return T{ clamp_float(v.x, lo, hi), clamp_float(v.y, lo, hi), clamp_float(v.z, lo, hi) };
    else return T{ clamp_float(v.x, lo, hi), clamp_float(v.y, lo, hi), clamp_float(v.z, lo, hi), clamp_float(v.w, lo, hi) };
}
} // namespace detail
// Float channels clamped to [0, 1] (saturate.h:95-111).
template <typename T>
struct SaturateFloat {
private:
    using SelfType = SaturateFloat<T>;

public:
    FK_UNARY_OPERATION(SaturateFloat, T, T)
    static_assert(std::is_same_v<VBase<T>, float>, "SaturateFloat only works with float base types.");
    FK_HD_STATIC OutputType exec(const InputType& input) { return detail::clamp_channels(input, 0.f, 1.f); }
};
// Float channels clamped to [0, maxDepthValue].
template <typename T, ColorDepth CD>
struct SaturateDepth {
private:
    using SelfType = SaturateDepth<T, CD>;

public:
    FK_UNARY_OPERATION(SaturateDepth, T, T)
    static_assert(std::is_same_v<VBase<T>, float>, "SaturateDepth only works with float base types.");
    FK_HD_STATIC OutputType exec(const InputType& input) {
        return detail::clamp_channels(input, 0.f, static_cast<float>(maxDepthValue<CD>));
    }
};
template <typename I, typename O, ColorDepth CD>
struct SaturateDenormalizePixel {
private:
    using SelfType = SaturateDenormalizePixel<I, O, CD>;

public:
    FK_UNARY_OPERATION(SaturateDenormalizePixel, I, O)
    static_assert(std::is_same_v<VBase<I>, float>, "SaturateDenormalizePixel only works with float base types.");
    FK_HD_STATIC OutputType exec(const InputType& input) { return DenormalizePixel<O, CD>::exec(SaturateFloat<I>::exec(input)); }
};
template <typename T, ColorDepth CD>
struct NormalizeColorRangeDepth {
private:
    using SelfType = NormalizeColorRangeDepth<T, CD>;

public:
    FK_UNARY_OPERATION(NormalizeColorRangeDepth, T, T)
    static_assert(std::is_floating_point_v<VBase<T>>, "NormalizeColorRangeDepth only works for floating point values");
    FK_HD_STATIC OutputType exec(const InputType& input) { return input * floatShiftFactor<CD>; }
};

// ---- YUV -> RGB ----------------------------------------------------------------------------------------------
// Input {Y, Cb, Cr} as stored.  Samples are shifted down to their depth's range, offset (chroma always, luma for
// bt601 only), multiplied by the matrix, then either saturated to the storage type and shifted back up, or (float
// outputs) scaled by the depth's float shift factor.  The alpha channel goes through the same last step.
template <PixelFormat PF, ColorRange CR, ColorPrimitives CP, bool ALPHA, typename ReturnType = YUVOutputPixelType<PF, ALPHA>>
struct ConvertYUVToRGB {
private:
    using SelfType = ConvertYUVToRGB<PF, CR, CP, ALPHA, ReturnType>;
    using Packed = PackedPixelType<PF>;
    static_assert(cn<Packed> == 3, "ConvertYUVToRGB takes three-channel YUV pixels");
    static_assert(cn<ReturnType> == (ALPHA ? 4 : 3), "ReturnType must have 4 channels with ALPHA, 3 without");

    // MxVFloat3 on a centred pixel with the matrix as compile-time constants, without the terms whose coefficient is
    // zero (two of the nine in every YCbCr -> RGB matrix).  The results are the same bits: the chroma differences are
    // finite, so such a term is +0 or -0, and the sum it would be added to is never -0 (luma comes from an integer, and
    // x - x is +0), so adding it changes nothing.
    static constexpr M3x3Float MATRIX = ccMatrix<CR, CP, ColorConversionDir::YCbCr2RGB>;
    template <int ROW>
    static constexpr float3 matrix_row() {
        if constexpr (ROW == 0) return MATRIX.x;
        else if constexpr (ROW == 1) return MATRIX.y;
        else return MATRIX.z;
    }
    template <int ROW>
    FK_HD_STATIC float row_times(const float3& v) {
        constexpr float3 row = matrix_row<ROW>();
        float sum = v.x * row.x;
        if constexpr (row.y != 0.f) sum = sum + v.y * row.y;
        if constexpr (row.z != 0.f) sum = sum + v.z * row.z;
        return sum;
    }

public:
    static constexpr ColorDepth CD = PixelFormatTraits<PF>::depth;
    FK_UNARY_OPERATION(ConvertYUVToRGB, Packed, ReturnType)

    FK_HD_STATIC OutputType exec(const InputType& input) {
        constexpr uint shift = shiftFactor<CD>;
        const InputType yuv = ShiftRight<InputType>::exec(input, shift);
        constexpr float chromaSub = subCoefficients<CD>.chroma;
        constexpr float lumaSub = CP == ColorPrimitives::bt601 ? subCoefficients<CD>.luma : 0.f;
        float3 centred{ static_cast<float>(yuv.x), yuv.y - chromaSub, yuv.z - chromaSub };
        if constexpr (CP == ColorPrimitives::bt601) centred.x = yuv.x - lumaSub;
        const float3 rgb{ row_times<0>(centred), row_times<1>(centred), row_times<2>(centred) };
        if constexpr (std::is_same_v<VBase<OutputType>, float>) {
            constexpr float scale = floatShiftFactor<CD>;
            if constexpr (ALPHA) {
                return OutputType{ rgb.x, rgb.y, rgb.z, static_cast<float>(maxDepthValue<CD>) } * scale;
            } else {
                return rgb * scale;
            }
        } else {
            const InputType stored = SaturateCast<float3, InputType>::exec(rgb);
            if constexpr (ALPHA) {
                return ShiftLeft<OutputType>::exec(OutputType{ stored.x, stored.y, stored.z, maxDepthValue<CD> }, shift);
            } else {
                return ShiftLeft<OutputType>::exec(stored, shift);
            }
        }
    }
};

// ---- memory layout of the supported formats --------------------------------------------------------------------
namespace detail {
// Semi-planar: a luma plane of `height` rows, then rows of interleaved chroma pairs, one pair per two pixels along x
// and per (1 << CHROMA_ROW_SHIFT) rows.  Packed 4:2:2: four samples per two pixels in one row.
template <PixelFormat PF>
struct YuvLayout {
    static constexpr bool supported = false;
};
template <bool U_FIRST, int CHROMA_ROW_SHIFT>
struct SemiPlanar {
    static constexpr bool supported = true;
    static constexpr bool semi_planar = true;
    static constexpr int u = U_FIRST ? 0 : 1, v = U_FIRST ? 1 : 0, row_shift = CHROMA_ROW_SHIFT;
};
template <int Y0, int Y1, int U, int V>
struct Packed422 {
    static constexpr bool supported = true;
    static constexpr bool semi_planar = false;
    static constexpr int y0 = Y0, y1 = Y1, u = U, v = V;
};
template <> struct YuvLayout<PixelFormat::NV12> : SemiPlanar<true, 1> {};
template <> struct YuvLayout<PixelFormat::NV21> : SemiPlanar<false, 1> {};
template <> struct YuvLayout<PixelFormat::P010> : SemiPlanar<true, 1> {};
template <> struct YuvLayout<PixelFormat::P210> : SemiPlanar<true, 0> {};
template <> struct YuvLayout<PixelFormat::UYVY> : Packed422<1, 3, 0, 2> {};
template <> struct YuvLayout<PixelFormat::Y210> : Packed422<0, 2, 1, 3> {};

template <typename Base>
FK_HD_CNST Base* yuv_row(Base* data, const uint pitch, const size_t row) {
    using Byte = std::conditional_t<std::is_const_v<Base>, const char, char>;
    return reinterpret_cast<Base*>(reinterpret_cast<Byte*>(data) + row * pitch);
}
} // namespace detail

template <PixelFormat PF>
class Image;

// One {Y, U, V} pixel per thread, chroma taken from the sample that covers the pixel (no chroma interpolation).
template <PixelFormat PF>
struct ReadYUV {
private:
    using SelfType = ReadYUV<PF>;
    using Layout = detail::YuvLayout<PF>;
    static_assert(Layout::supported, "ReadYUV: pixel format not supported");

public:
    FK_STATIC_STRUCT(ReadYUV, SelfType)
    using PixelBaseType = ColorDepthPixelBaseType<PixelFormatTraits<PF>::depth>;
    using ParamsType = RawImage<PF>;
    using ReadDataType = PixelBaseType;
    using OutputType = ColorDepthPixelType<PixelFormatTraits<PF>::depth>;
    using InstanceType = ReadType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Read<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;

    FK_HD_STATIC OutputType exec(const Point& thread, const ParamsType& params) {
        const PixelBaseType* const data = params.data.data;
        const uint pitch = params.data.dims.pitch;
        if constexpr (Layout::semi_planar) {
            const PixelBaseType luma = detail::yuv_row(data, pitch, thread.y)[thread.x];
            const PixelBaseType* const pair =
                detail::yuv_row(data, pitch, static_cast<size_t>(params.height) + (thread.y >> Layout::row_shift)) + 2 * (thread.x >> 1);
            return OutputType{ luma, pair[Layout::u], pair[Layout::v] };
        } else {
            const PixelBaseType* const quad = detail::yuv_row(data, pitch, thread.y) + 4 * (thread.x >> 1);
            return OutputType{ quad[(thread.x & 1) ? Layout::y1 : Layout::y0], quad[Layout::u], quad[Layout::v] };
        }
    }
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return exec(thread, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return opData.params.width; }
    FK_HD_STATIC uint num_elems_y(const Point&, const OperationDataType& opData) { return opData.params.height; }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) { return { opData.params.width, opData.params.height, 1u }; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    static inline InstantiableType build(const Image<PF>& image);
};

// One {Y, U, V} pixel per thread into a raw YUV image.  Each chroma sample is written by exactly one of the pixels
// it covers: the even one(s) for NV12/P010/P210/UYVY/Y210 (color_conversion.h:425-437,454-483).  For NV21 the
// reference lets all four covered pixels write (:446); the last of them in its host loop, the odd-x odd-y pixel, is
// the one that writes here.
template <PixelFormat PF>
struct WriteYUV {
private:
    using SelfType = WriteYUV<PF>;
    using Layout = detail::YuvLayout<PF>;
    static_assert(Layout::supported, "WriteYUV: pixel format not supported");

public:
    FK_STATIC_STRUCT(WriteYUV, SelfType)
    using PixelBaseType = ColorDepthPixelBaseType<PixelFormatTraits<PF>::depth>;
    using ParamsType = RawImage<PF>;
    using InputType = ColorDepthPixelType<PixelFormatTraits<PF>::depth>;
    using WriteDataType = PixelBaseType;
    using InstanceType = WriteType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Write<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;

    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const ParamsType& params) {
        PixelBaseType* const data = params.data.data;
        const uint pitch = params.data.dims.pitch;
        const bool even_x = (thread.x & 1) == 0;
        if constexpr (Layout::semi_planar) {
            detail::yuv_row(data, pitch, thread.y)[thread.x] = input.x;
            bool writes_chroma = even_x;
            if constexpr (PF == PixelFormat::NV21) writes_chroma = (thread.x & 1) && (thread.y & 1);
            else if constexpr (Layout::row_shift == 1) writes_chroma = even_x && (thread.y & 1) == 0;
            if (writes_chroma) {
                PixelBaseType* const pair =
                    detail::yuv_row(data, pitch, static_cast<size_t>(params.height) + (thread.y >> Layout::row_shift)) + 2 * (thread.x >> 1);
                pair[Layout::u] = input.y;
                pair[Layout::v] = input.z;
            }
        } else {
            PixelBaseType* const quad = detail::yuv_row(data, pitch, thread.y) + 4 * (thread.x >> 1);
            if (even_x) {
                quad[Layout::y0] = input.x;
                quad[Layout::u] = input.y;
                quad[Layout::v] = input.z;
            } else {
                quad[Layout::y1] = input.x;
            }
        }
    }
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const OperationDataType& opData) { exec(thread, input, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return opData.params.width; }
    FK_HD_STATIC uint num_elems_y(const Point&, const OperationDataType& opData) { return opData.params.height; }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) { return { opData.params.width, opData.params.height, 1u }; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    static inline InstantiableType build(const Image<PF>& image);
};

// Owner of a YUV image: one 2D buffer of (width * rf.width_f) x (height * rf.height_f) base-type elements.
template <PixelFormat PF>
class Image {
public:
    using BaseType = ColorDepthPixelBaseType<PixelFormatTraits<PF>::depth>;
    static constexpr PixelFormat pixelFormat = PF;

private:
    Ptr<ND::_2D, BaseType> data;
    uint width{ 0 };
    uint height{ 0 };
    static constexpr ResolutionFactors rf = PixelFormatTraits<PF>::rf;

public:
    Image() {}
    Image(const Ptr<ND::_2D, BaseType>& data_, const uint& width_, const uint& height_) : data(data_), width(width_), height(height_) {}
    Image(const uint width_, const uint height_, const MemType& memType = defaultMemType, const int deviceID = 0)
        : data(PtrDims<ND::_2D>(static_cast<uint>(width_ * rf.width_f), static_cast<uint>(height_ * rf.height_f)), memType, deviceID),
          width(width_), height(height_) {}

    uint imageWidth() const { return width; }
    uint imageHeight() const { return height; }
    RawImage<PF> ptr() const { return RawImage<PF>{ data.ptr(), width, height }; }
    RawImage<PF> operator()() const { return ptr(); }
    Ptr<ND::_2D, BaseType> getData() const { return data; }

    // A view of newWidth x newHeight pixels at p.  Meaningful for the packed formats; in a semi-planar image the
    // chroma plane of the view no longer follows its luma rows (as in the reference, image.h:62-68).
    Image<PF> crop(const Point& p, const uint& newWidth, const uint& newHeight) {
        const Point dataPoint(static_cast<int>(p.x * rf.width_f), static_cast<int>(p.y * rf.height_f));
        const PtrDims<ND::_2D> newDims(static_cast<uint>(newWidth * rf.width_f), static_cast<uint>(newHeight * rf.height_f), data.dims().pitch);
        return Image<PF>(data.crop(dataPoint, newDims), newWidth, newHeight);
    }

    void uploadTo(Image& other, fkrt_stream stream = nullptr) { data.uploadTo(other.data, stream); }
    void downloadTo(Image& other, fkrt_stream stream = nullptr) { data.downloadTo(other.data, stream); }
    void upload(Stream& stream) { data.upload(stream); }
    void download(Stream& stream) { data.download(stream); }

    // Host read of one pixel (host or pinned memory only).
    VectorType_t<BaseType, static_cast<int>(PixelFormatTraits<PF>::cn)> readAt(const Point& p) const {
        if (data.getMemType() == MemType::Device) throw std::runtime_error("This is a device image, cannot read pixels on the host.");
        RawImage<PF> host = ptr();
        host.data = data.ptrPinned();
        return ReadYUV<PF>::exec(p, host);
    }
};

template <PixelFormat PF>
inline typename ReadYUV<PF>::InstantiableType ReadYUV<PF>::build(const Image<PF>& image) { return InstantiableType{ { image.ptr() } }; }
template <PixelFormat PF>
inline typename WriteYUV<PF>::InstantiableType WriteYUV<PF>::build(const Image<PF>& image) { return InstantiableType{ { image.ptr() } }; }

} // namespace fk
#endif
