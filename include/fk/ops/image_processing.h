// Image operations on the fused Transform path: ColorConversion, Crop, Interpolate, Resize.
// Semantics follow the reference's algorithms/image_processing/color_conversion.h:47-77,516-613, crop.h:23-90,
// interpolation.h:49-97 and resize.h:42-348.  The bilinear row index is taken from the y coordinate, as the
// reference's device branch does (interpolation.h:66-67); defining FK_INTERPOLATE_Y1_FROM_X selects its host
// branch (:69-70), which takes it from the x coordinate.
#ifndef FK_OPS_IMAGE_PROCESSING_H
#define FK_OPS_IMAGE_PROCESSING_H

#include "fk/ops/arithmetic.h"
#include "fk/ops/memory_operations.h"

namespace fk {

// ---- color conversion ----------------------------------------------------------------------------------------
enum class ColorConversionCodes {
    COLOR_BGR2BGRA = 0, COLOR_RGB2RGBA = COLOR_BGR2BGRA,
    COLOR_BGRA2BGR = 1, COLOR_RGBA2RGB = COLOR_BGRA2BGR,
    COLOR_BGR2RGBA = 2, COLOR_RGB2BGRA = COLOR_BGR2RGBA,
    COLOR_RGBA2BGR = 3, COLOR_BGRA2RGB = COLOR_RGBA2BGR,
    COLOR_BGR2RGB = 4, COLOR_RGB2BGR = COLOR_BGR2RGB,
    COLOR_BGRA2RGBA = 5, COLOR_RGBA2BGRA = COLOR_BGRA2RGBA,
    COLOR_BGR2GRAY = 6,
    COLOR_RGB2GRAY = 7,
    COLOR_BGRA2GRAY = 10,
    COLOR_RGBA2GRAY = 11
};
enum class ColorDepth { p8bit = 0, p10bit = 1, p12bit = 2, f24bit = 3 };

// CCIR 601 luma of the first three channels as stored, rounded to nearest even for integer outputs
// (color_conversion.h:47-77).
enum class GrayFormula { CCIR_601 };

template <typename I, typename O = VBase<I>, GrayFormula GF = GrayFormula::CCIR_601>
struct RGB2Gray {
private:
    using SelfType = RGB2Gray<I, O, GF>;

public:
    FK_UNARY_OPERATION(RGB2Gray, I, O)
    static_assert(cn<I> >= 3, "RGB2Gray needs three or more channels");
    FK_HD_STATIC OutputType exec(const InputType& input) {
        const float gray = (input.x * 0.299f + input.y * 0.587f) + input.z * 0.114f;
        if constexpr (std::is_integral_v<O>) {
            return static_cast<O>(__builtin_rintf(gray));
        } else {
            return static_cast<O>(gray);
        }
    }
};

// Opaque alpha appended to a 3-channel pixel.
template <typename I, ColorDepth CD = ColorDepth::p8bit>
struct AddOpaqueAlpha {
private:
    using SelfType = AddOpaqueAlpha<I, CD>;
    using O4 = VectorType_t<VBase<I>, 4>;

public:
    FK_UNARY_OPERATION(AddOpaqueAlpha, I, O4)
    static_assert(cn<I> == 3, "AddOpaqueAlpha takes a 3-channel pixel");
    FK_HD_STATIC OutputType exec(const InputType& input) {
        constexpr VBase<I> alpha = std::is_floating_point_v<VBase<I>> ? static_cast<VBase<I>>(1)
                                   : CD == ColorDepth::p8bit          ? static_cast<VBase<I>>(255)
                                   : CD == ColorDepth::p10bit         ? static_cast<VBase<I>>(1023)
                                                                      : static_cast<VBase<I>>(4095);
        return O4{ input.x, input.y, input.z, alpha };
    }
};

// A given alpha appended to a 3-channel pixel (color_conversion.h:29-40).
template <typename I, VBase<I> alpha>
struct StaticAddAlpha {
private:
    using SelfType = StaticAddAlpha<I, alpha>;
    using O4 = VectorType_t<VBase<I>, 4>;

public:
    FK_UNARY_OPERATION(StaticAddAlpha, I, O4)
    static_assert(cn<I> == 3, "StaticAddAlpha takes a 3-channel pixel");
    FK_HD_STATIC OutputType exec(const InputType& input) { return O4{ input.x, input.y, input.z, alpha }; }
};

namespace detail {
template <ColorConversionCodes CODE, typename I, typename O, ColorDepth CD>
struct ColorConversionType {
    static_assert(sizeof(I) == 0, "Color conversion code not supported");
};
template <typename I, typename O, ColorDepth CD>
struct ColorConversionType<ColorConversionCodes::COLOR_BGR2BGRA, I, O, CD> { using type = AddOpaqueAlpha<I, CD>; };
template <typename I, typename O, ColorDepth CD>
struct ColorConversionType<ColorConversionCodes::COLOR_BGRA2BGR, I, O, CD> { using type = Discard<I, VectorType_t<VBase<I>, 3>>; };
template <typename I, typename O, ColorDepth CD>
struct ColorConversionType<ColorConversionCodes::COLOR_BGR2RGBA, I, O, CD> { using type = FusedOperation<VectorReorder<I, 2, 1, 0>, AddOpaqueAlpha<I, CD>>; };
template <typename I, typename O, ColorDepth CD>
struct ColorConversionType<ColorConversionCodes::COLOR_RGBA2BGR, I, O, CD> { using type = FusedOperation<VectorReorder<I, 2, 1, 0, 3>, Discard<I, VectorType_t<VBase<I>, 3>>>; };
template <typename I, typename O, ColorDepth CD>
struct ColorConversionType<ColorConversionCodes::COLOR_BGR2RGB, I, O, CD> { using type = VectorReorder<I, 2, 1, 0>; };
template <typename I, typename O, ColorDepth CD>
struct ColorConversionType<ColorConversionCodes::COLOR_BGRA2RGBA, I, O, CD> { using type = VectorReorder<I, 2, 1, 0, 3>; };
template <typename I, typename O, ColorDepth CD>
struct ColorConversionType<ColorConversionCodes::COLOR_RGB2GRAY, I, O, CD> { using type = RGB2Gray<I, O>; };
template <typename I, typename O, ColorDepth CD>
struct ColorConversionType<ColorConversionCodes::COLOR_RGBA2GRAY, I, O, CD> { using type = RGB2Gray<I, O>; };
template <typename I, typename O, ColorDepth CD>
struct ColorConversionType<ColorConversionCodes::COLOR_BGR2GRAY, I, O, CD> { using type = FusedOperation<VectorReorder<I, 2, 1, 0>, RGB2Gray<I, O>>; };
template <typename I, typename O, ColorDepth CD>
struct ColorConversionType<ColorConversionCodes::COLOR_BGRA2GRAY, I, O, CD> { using type = FusedOperation<VectorReorder<I, 2, 1, 0, 3>, RGB2Gray<I, O>>; };
} // namespace detail

template <ColorConversionCodes CODE, typename I, typename O, ColorDepth CD = ColorDepth::p8bit>
using ColorConversion = typename detail::ColorConversionType<CODE, I, O, CD>::type;

// ---- crop ------------------------------------------------------------------------------------------------------
// Reads the back operation at thread + rect origin; z is dropped (crop.h:35-38).
template <typename BackIOp_ = void>
struct Crop : BatchBuilders<Crop<BackIOp_>> {
private:
    using SelfType = Crop<BackIOp_>;

public:
    FK_STATIC_STRUCT(Crop, SelfType)
    using ReadDataType = typename BackIOp_::Operation::OutputType;
    using OutputType = typename BackIOp_::Operation::OutputType;
    using ParamsType = Rect;
    using BackIOp = BackIOp_;
    using InstanceType = ReadBackType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = ReadBack<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;

    FK_HD_STATIC OutputType exec(const Point& thread, const ParamsType& params, const BackIOp& backIOp) {
        const Point newThread(static_cast<int>(thread.x + params.x), static_cast<int>(thread.y + params.y));
        return BackIOp::Operation::exec(newThread, backIOp);
    }
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return exec(thread, opData.params, opData.backIOp); }
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return static_cast<uint>(opData.params.width); }
    FK_HD_STATIC uint num_elems_y(const Point&, const OperationDataType& opData) { return static_cast<uint>(opData.params.height); }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return { num_elems_x(Point(), opData), num_elems_y(Point(), opData), 1u };
    }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    FK_HD_STATIC InstantiableType build(const BackIOp& backIOp, const Rect& rect) { return InstantiableType{ { rect, backIOp } }; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return InstantiableType{ { params, backIOp } }; }
    using BatchBuilders<SelfType>::build;
};

// Builder form: Crop<>::build(rect) waits for the read that precedes it in a .then() chain.
template <>
struct Crop<void> : BatchBuilders<Crop<void>> {
private:
    using SelfType = Crop<void>;

public:
    FK_STATIC_STRUCT(Crop, SelfType)
    static constexpr bool BUILDER_ONLY = true; // executes only once completed with its back read
    using ReadDataType = NullType;
    using OutputType = NullType;
    using ParamsType = Rect;
    using BackIOp = NullType;
    using InstanceType = ReadBackType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = ReadBack<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;

    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return static_cast<uint>(opData.params.width); }
    FK_HD_STATIC uint num_elems_y(const Point&, const OperationDataType& opData) { return static_cast<uint>(opData.params.height); }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC InstantiableType build(const Rect& rect) { return InstantiableType{ { rect, {} } }; }
    template <typename RealBackIOp, std::enable_if_t<isAnyReadType<RealBackIOp>, int> = 0>
    FK_HD_STATIC auto build(const RealBackIOp& backIOp, const InstantiableType& self) {
        return Crop<RealBackIOp>::build(backIOp, self.params);
    }
    template <typename RealBackIOp, std::enable_if_t<isAnyReadType<RealBackIOp>, int> = 0>
    FK_HD_STATIC auto build(const RealBackIOp& backIOp, const Rect& rect) {
        return Crop<RealBackIOp>::build(backIOp, rect);
    }
    using BatchBuilders<SelfType>::build;
};

// ---- interpolation ---------------------------------------------------------------------------------------------
enum class InterpolationType { INTER_LINEAR = 1, NONE = 17 };

template <InterpolationType INTER_T>
struct InterpolationParameters {};
template <>
struct InterpolationParameters<InterpolationType::INTER_LINEAR> {
    Size src_size;
};

namespace detail {
// The 2x2 footprint of a bilinear sample: integer corners (x2r, y2r clamped to the source) and the four
// weights, which use the unclamped x1+1, y1+1 (interpolation.h:61-96).
struct BilinearTaps {
    int x1, y1, x2r, y2r;
    float wa, wb, wc, wd;
};
// floor() as an int, exact for every float that fits one (usable in constant expressions)
FK_HD_CNST int floor_to_int(const float v) {
    const int t = static_cast<int>(v);
    return static_cast<float>(t) > v ? t - 1 : t;
}
FK_HD_CNST BilinearTaps bilinear_taps(const float src_x, const float src_y, const Size& srcSize) {
#if defined(__HIP_DEVICE_COMPILE__)
    if (!__builtin_is_constant_evaluated()) {
        // The same values with fewer conversions: floor() is one instruction, and for |x| < 2^24 (any image) the float
        // of x1 is floor(src_x) itself and the float of x1 + 1 is floor(src_x) + 1.
        const float x1f = __builtin_floorf(src_x);
#ifdef FK_INTERPOLATE_Y1_FROM_X
        const float y1f = x1f;
#else
        const float y1f = __builtin_floorf(src_y);
#endif
        const int x1 = static_cast<int>(x1f), y1 = static_cast<int>(y1f);
        // src_x - x1 is exact (x1 = floor(src_x) is at least half of src_x, or zero), so x2 - src_x, one rounding of
        // 1 - (src_x - x1), is 1.0f minus that difference; the same for y
        const float fx = src_x - x1f, fy = src_y - y1f;
        const float gx = 1.0f - fx;
#ifdef FK_INTERPOLATE_Y1_FROM_X
        const float gy = (y1f + 1.0f) - src_y; // y1 is not the floor of src_y here: the difference above may be rounded
#else
        const float gy = 1.0f - fy;
#endif
        BilinearTaps t{};
        t.x1 = x1;
        t.y1 = y1;
        t.x2r = x1 + 1 < srcSize.width - 1 ? x1 + 1 : srcSize.width - 1;
        t.y2r = y1 + 1 < srcSize.height - 1 ? y1 + 1 : srcSize.height - 1;
        t.wa = gx * gy;
        t.wb = fx * gy;
        t.wc = gx * fy;
        t.wd = fx * fy;
        return t;
    }
#endif
    const int x1 = floor_to_int(src_x);
#ifdef FK_INTERPOLATE_Y1_FROM_X
    const int y1 = floor_to_int(src_x);
#else
    const int y1 = floor_to_int(src_y);
#endif
    const int x2 = x1 + 1;
    const int y2 = y1 + 1;
    BilinearTaps t{};
    t.x1 = x1;
    t.y1 = y1;
    t.x2r = x2 < srcSize.width - 1 ? x2 : srcSize.width - 1;
    t.y2r = y2 < srcSize.height - 1 ? y2 : srcSize.height - 1;
    t.wa = (x2 - src_x) * (y2 - src_y);
    t.wb = (src_x - x1) * (y2 - src_y);
    t.wc = (x2 - src_x) * (src_y - y1);
    t.wd = (src_x - x1) * (src_y - y1);
    return t;
}
// ((a*wa + b*wb) + c*wc) + d*wd per channel, in this order.
template <typename Pixel>
FK_HD_CNST auto bilinear_blend(const Pixel& a, const Pixel& b, const Pixel& c, const Pixel& d, const BilinearTaps& t) {
    return (a * t.wa) + (b * t.wb) + (c * t.wc) + (d * t.wd);
}
} // namespace detail

template <InterpolationType INTER_T, typename BackIOp_ = void>
struct Interpolate;

template <typename BackIOp_>
struct Interpolate<InterpolationType::INTER_LINEAR, BackIOp_> {
private:
    using SelfType = Interpolate<InterpolationType::INTER_LINEAR, BackIOp_>;
    using ReadOutputType = typename BackIOp_::Operation::OutputType;

public:
    FK_STATIC_STRUCT(Interpolate, SelfType)
    using InputType = float2;
    using ParamsType = InterpolationParameters<InterpolationType::INTER_LINEAR>;
    using BackIOp = BackIOp_;
    using OutputType = VectorType_t<float, cn<ReadOutputType>>;
    using InstanceType = TernaryType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Ternary<SelfType>;
    static constexpr bool IS_FUSED_OP = false;

    FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params, const BackIOp& backIOp) {
        const detail::BilinearTaps t = detail::bilinear_taps(input.x, input.y, params.src_size);
        using ReadOperation = typename BackIOp::Operation;
        const ReadOutputType a = ReadOperation::exec(Point(t.x1, t.y1), backIOp);
        const ReadOutputType b = ReadOperation::exec(Point(t.x2r, t.y1), backIOp);
        const ReadOutputType c = ReadOperation::exec(Point(t.x1, t.y2r), backIOp);
        const ReadOutputType d = ReadOperation::exec(Point(t.x2r, t.y2r), backIOp);
        return detail::bilinear_blend(a, b, c, d, t);
    }
    FK_HD_STATIC OutputType exec(const InputType& input, const OperationDataType& opData) { return exec(input, opData.params, opData.backIOp); }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return InstantiableType{ { params, backIOp } }; }
};

// ---- resize ----------------------------------------------------------------------------------------------------
enum class AspectRatio { PRESERVE_AR = 0, IGNORE_AR = 1, PRESERVE_AR_RN_EVEN = 2, PRESERVE_AR_LEFT = 3 };

template <InterpolationType IType, AspectRatio AR = AspectRatio::IGNORE_AR, typename T = void>
struct ResizeReadParams {
    Size dstSize;
    float2 src_conv_factors;
    InterpolationParameters<IType> params;
    int x1, y1; // top left of the region that holds the resized image
    int x2, y2; // bottom right
    T defaultValue;
};
template <InterpolationType IType>
struct ResizeReadParams<IType, AspectRatio::IGNORE_AR, void> {
    Size dstSize;
    float2 src_conv_factors;
    InterpolationParameters<IType> params;
};

template <AspectRatio AR, typename T = void>
struct IncompleteResizeReadParams {
    Size dstSize;
    T defaultValue;
};
template <AspectRatio AR>
struct IncompleteResizeReadParams<AR, void> {
    Size dstSize;
};

template <InterpolationType IType, AspectRatio AR = AspectRatio::IGNORE_AR, typename BackIOp_ = void>
struct Resize : BatchBuilders<Resize<IType, AR, BackIOp_>> {
private:
    using SelfType = Resize<IType, AR, BackIOp_>;

public:
    FK_STATIC_STRUCT(Resize, SelfType)
    using InterpolateOutputType = typename Interpolate<IType, BackIOp_>::OutputType;
    using ReadDataType = typename BackIOp_::Operation::OutputType;
    using OutputType = InterpolateOutputType;
    using ParamsType = ResizeReadParams<IType, AR, std::conditional_t<AR == AspectRatio::IGNORE_AR, void, InterpolateOutputType>>;
    using BackIOp = BackIOp_;
    using InstanceType = ReadBackType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = ReadBack<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;
    static constexpr AspectRatio ASPECT = AR;

    FK_HD_STATIC OutputType exec(const Point& thread, const ParamsType& params, const BackIOp& backIOp) {
        if constexpr (AR == AspectRatio::IGNORE_AR) {
            return exec_resize(thread, params, backIOp);
        } else {
            if (thread.x >= params.x1 && thread.x <= params.x2 && thread.y >= params.y1 && thread.y <= params.y2) {
                return exec_resize(Point(thread.x - params.x1, thread.y - params.y1, thread.z), params, backIOp);
            } else {
                return params.defaultValue;
            }
        }
    }
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return exec(thread, opData.params, opData.backIOp); }
    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType& opData) { return static_cast<uint>(opData.params.dstSize.width); }
    FK_HD_STATIC uint num_elems_y(const Point&, const OperationDataType& opData) { return static_cast<uint>(opData.params.dstSize.height); }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return { num_elems_x(Point(), opData), num_elems_y(Point(), opData), 1u };
    }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return InstantiableType{ { params, backIOp } }; }

    // IGNORE_AR: stretch the back read to dstSize (resize.h:105-119).  Conversion factors are computed in double.
    template <AspectRatio AR_ = AR, std::enable_if_t<AR_ == AspectRatio::IGNORE_AR, int> = 0>
    static inline constexpr InstantiableType build(const BackIOp& backIOp, const Size& dstSize) {
        const Size srcSize = Num_elems<BackIOp>::size(Point(), backIOp);
        const double cfx = static_cast<double>(dstSize.width) / static_cast<double>(srcSize.width);
        const double cfy = static_cast<double>(dstSize.height) / static_cast<double>(srcSize.height);
        const ParamsType resizeParams{ dstSize, { static_cast<float>(1.0 / cfx), static_cast<float>(1.0 / cfy) }, { srcSize } };
        return InstantiableType{ { resizeParams, backIOp } };
    }
    // PRESERVE_AR*: fit inside dstSize keeping the aspect ratio, centred (or left-aligned), rest = background
    // (resize.h:121-166, target size :196-221).
    template <AspectRatio AR_ = AR, std::enable_if_t<AR_ != AspectRatio::IGNORE_AR, int> = 0>
    static inline constexpr InstantiableType build(const BackIOp& backIOp, const Size& dstSize, const OutputType& backgroundValue) {
        const Size srcSize = Num_elems<BackIOp>::size(Point(), backIOp);
        const Size targetSize = compute_target_size(srcSize, dstSize);
        const double cfx = static_cast<double>(targetSize.width) / srcSize.width;
        const double cfy = static_cast<double>(targetSize.height) / srcSize.height;
        const int x1 = AR_ == AspectRatio::PRESERVE_AR_LEFT ? 0 : static_cast<int>((dstSize.width - targetSize.width) / 2);
        const int y1 = static_cast<int>((dstSize.height - targetSize.height) / 2);
        const ParamsType resizeParams{ dstSize,
                                       { static_cast<float>(1.0 / cfx), static_cast<float>(1.0 / cfy) },
                                       { srcSize },
                                       x1, y1, x1 + targetSize.width - 1, y1 + targetSize.height - 1,
                                       backgroundValue };
        return InstantiableType{ { resizeParams, backIOp } };
    }
    using BatchBuilders<SelfType>::build;

private:
    FK_HD_STATIC OutputType exec_resize(const Point& thread, const ParamsType& params, const BackIOp& backIOp) {
        const float src_x = thread.x * params.src_conv_factors.x;
        const float src_y = thread.y * params.src_conv_factors.y;
        return Interpolate<IType, BackIOp>::exec(float2{ src_x, src_y }, params.params, backIOp);
    }
    static inline constexpr Size compute_target_size(const Size& srcSize, const Size& dstSize) {
        const float scaleFactor = dstSize.height / static_cast<float>(srcSize.height);
        const int targetHeight = dstSize.height;
        const int targetWidth = static_cast<int>(cxp::round(scaleFactor * srcSize.width));
        if constexpr (AR == AspectRatio::PRESERVE_AR_RN_EVEN) {
            const int evenWidth = targetWidth - (targetWidth % 2);
            if (evenWidth > dstSize.width) {
                const float scaleByWidth = dstSize.width / static_cast<float>(srcSize.width);
                const int h = static_cast<int>(cxp::round(scaleByWidth * srcSize.height));
                return Size(dstSize.width, h - (h % 2));
            }
            return Size(evenWidth, targetHeight);
        } else {
            if (targetWidth > dstSize.width) {
                const float scaleByWidth = dstSize.width / static_cast<float>(srcSize.width);
                return Size(dstSize.width, static_cast<int>(cxp::round(scaleByWidth * srcSize.height)));
            }
            return Size(targetWidth, targetHeight);
        }
    }
};

// Builder form with parameters: Resize<...>::build(dstSize[, background]) waits for its back read.
template <InterpolationType IType, AspectRatio AR, typename T>
struct Resize<IType, AR, TypeList<void, T>> : BatchBuilders<Resize<IType, AR, TypeList<void, T>>> {
private:
    using SelfType = Resize<IType, AR, TypeList<void, T>>;

public:
    FK_STATIC_STRUCT(Resize, SelfType)
    static constexpr bool BUILDER_ONLY = true;
    using ReadDataType = NullType;
    using OutputType = std::conditional_t<std::is_void_v<T>, NullType, T>;
    using ParamsType = IncompleteResizeReadParams<AR, T>;
    using BackIOp = NullType;
    using InstanceType = ReadBackType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = ReadBack<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;

    FK_HD_STATIC uint num_elems_x(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC uint num_elems_y(const Point&, const OperationDataType&) { return 1; }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType&) { return 1; }

    template <typename U = T, std::enable_if_t<std::is_void_v<U>, int> = 0>
    static inline constexpr InstantiableType build(const Size& dstSize) { return InstantiableType{ { { dstSize }, {} } }; }
    template <typename U = T, std::enable_if_t<!std::is_void_v<U>, int> = 0>
    static inline constexpr InstantiableType build(const Size& dstSize, const U& backgroundValue) {
        return InstantiableType{ { { dstSize, backgroundValue }, {} } };
    }
    // completion with the read that precedes it
    template <typename ReadIOp, std::enable_if_t<isAnyReadType<ReadIOp>, int> = 0>
    static inline constexpr auto build(const ReadIOp& readIOp, const InstantiableType& self) {
        if constexpr (std::is_void_v<T>) {
            return Resize<IType, AR, ReadIOp>::build(readIOp, self.params.dstSize);
        } else {
            using Out = typename Resize<IType, AR, ReadIOp>::OutputType;
            return Resize<IType, AR, ReadIOp>::build(readIOp, self.params.dstSize, detail::cast_channels<Out>(self.params.defaultValue));
        }
    }
    using BatchBuilders<SelfType>::build;
};

// Entry form: Resize<IType, AR>::build(...) with no back read named in the type.
template <InterpolationType IType, AspectRatio AR>
struct Resize<IType, AR, void> {
private:
    using SelfType = Resize<IType, AR, void>;

public:
    FK_STATIC_STRUCT(Resize, SelfType)
    using InstanceType = ReadBackType;
    static constexpr bool BUILDER_ONLY = true;

    template <typename BF, AspectRatio AR_ = AR, std::enable_if_t<AR_ == AspectRatio::IGNORE_AR && isAnyReadType<BF>, int> = 0>
    static inline constexpr auto build(const BF& backIOp, const Size& dstSize) {
        return Resize<IType, AR_, BF>::build(backIOp, dstSize);
    }
    template <typename BF, AspectRatio AR_ = AR, std::enable_if_t<AR_ != AspectRatio::IGNORE_AR && isAnyReadType<BF>, int> = 0>
    static inline constexpr auto build(const BF& backIOp, const Size& dstSize, const typename Resize<IType, AR_, BF>::OutputType& backgroundValue) {
        return Resize<IType, AR_, BF>::build(backIOp, dstSize, backgroundValue);
    }
    template <AspectRatio AR_ = AR, std::enable_if_t<AR_ == AspectRatio::IGNORE_AR, int> = 0>
    static inline constexpr auto build(const Size& dstSize) {
        return Resize<IType, AR_, TypeList<void, void>>::build(dstSize);
    }
    template <typename T, AspectRatio AR_ = AR, std::enable_if_t<AR_ != AspectRatio::IGNORE_AR && !isAnyReadType<T>, int> = 0>
    static inline constexpr auto build(const Size& dstSize, const T& backgroundValue) {
        return Resize<IType, AR_, TypeList<void, T>>::build(dstSize, backgroundValue);
    }
    template <typename T>
    static inline constexpr auto build(const RawPtr<ND::_2D, T>& input, const Size& dSize, const double& fx, const double& fy) {
        using ReadIOp = Read<PerThreadRead<ND::_2D, T>>;
        const ReadIOp readIOp = PerThreadRead<ND::_2D, T>::build(input);
        if (dSize.width != 0 && dSize.height != 0) {
            return Resize<IType, AR, ReadIOp>::build(readIOp, dSize);
        }
        const Size computed(SaturateCast<double, int>::exec(input.dims.width * fx), SaturateCast<double, int>::exec(input.dims.height * fy));
        return Resize<IType, AR, ReadIOp>::build(readIOp, computed);
    }
    // one plane per array element
    template <size_t BATCH_N, typename First, typename... Arrays>
    static inline constexpr auto build(const std::array<First, BATCH_N>& first, const Arrays&... arrays) {
        return BatchRead<BATCH_N, PlanePolicy::PROCESS_ALL>::build(BatchOperation::build_batch<SelfType>(first, arrays...));
    }
    template <size_t BATCH_N, typename DefaultValueType, typename First, typename... Arrays>
    static inline constexpr auto build(const int& usedPlanes, const DefaultValueType& defaultValue,
                                       const std::array<First, BATCH_N>& first, const Arrays&... arrays) {
        return BatchRead<BATCH_N, PlanePolicy::CONDITIONAL_WITH_DEFAULT>::build(
            BatchOperation::build_batch<SelfType>(first, arrays...), usedPlanes, defaultValue);
    }
};

} // namespace fk
#endif
