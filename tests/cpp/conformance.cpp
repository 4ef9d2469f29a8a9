// Host-side conformance of the fk:: operator API: type identities, sizes and values that user code written against
// the Fused Kernel Library relies on (the reference pins the same facts in its compile-time tests: tests/algorithm/
// test_crop.h:28-45, tests/operation/test_instantiable_operations.h:46-226, tests/operation/test_fused_operation.h:
// 49-116, tests/operation/test_operation_types.h:56-182, tests/data/test_rect.h:19-39, tests/data/test_ptr_nd.h:44-108).
// Needs no GPU: everything here is compile-time or host memory.  Exit code 0 = pass.
#include <fused_kernel/fused_kernel.h>
#include <fused_kernel/fused_kernel.cuh> // the spelling the reference's README still uses
#include <fused_kernel/algorithms/image_processing/resize.cuh>

#include <cstdio>
#include <cstring>

using namespace fk;

#define EXPECT(cond)                                                                                                   \
    do {                                                                                                               \
        if (!(cond)) {                                                                                                 \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);                                              \
            ++failures;                                                                                                \
        }                                                                                                              \
    } while (0)

// ---- vector types and operators -------------------------------------------------------------------------------
static_assert(sizeof(uchar3) == 3 && sizeof(uchar4) == 4 && alignof(uchar4) == 4 && sizeof(float3) == 12 && alignof(float3) == 4);
static_assert(sizeof(float2) == 8 && alignof(float2) == 8 && sizeof(float4) == 16 && alignof(float4) == 16 && alignof(short4) == 8);
static_assert(cn<uchar3> == 3 && cn<float> == 1 && cn<const uchar3> == 1);
static_assert(std::is_same_v<VBase<float4>, float> && std::is_same_v<VectorType_t<float, 3>, float3> && std::is_same_v<VectorType_t<uchar, 1>, uchar>);
static_assert(std::is_same_v<decltype(uchar3{} * uchar3{}), int3>, "integer promotion per channel");
static_assert(std::is_same_v<decltype(uchar3{} * 2.f), float3> && std::is_same_v<decltype(uchar4{} * 2), int4>);
static_assert(std::is_same_v<decltype(float3{} == float3{}), bool3>);
static_assert((make_<float3>(1, 2, 3) + make_set<float3>(1.f)).z == 4.f);
static_assert((uchar3{ 200, 100, 7 } * uchar3{ 2, 2, 2 }).x == 400, "no wrap-around: channels promote to int");

// ---- kinds ---------------------------------------------------------------------------------------------------
using ReadU3 = PerThreadRead<ND::_2D, uchar3>;
static_assert(isReadType<ReadU3> && isReadType<Read<ReadU3>> && !isReadBackType<ReadU3> && isAnyReadType<Crop<Read<ReadU3>>>);
static_assert(isReadBackType<Crop<Read<ReadU3>>> && isReadBackType<Crop<>> && !isCompleteOperation<Crop<>> && isCompleteOperation<Crop<Read<ReadU3>>>);
static_assert(isBinaryType<Mul<float3>> && isUnaryType<Cast<uchar3, float3>> && isWriteType<TensorWrite<float3>> && isComputeType<Mul<float>>);
static_assert(allUnaryTypes<Cast<int, float>, Cast<float, int>> && notAllUnaryTypes<Cast<int, float>, Mul<float>>);
static_assert(noneWriteType<ReadU3, Mul<float3>> && !noneAnyWriteType<ReadU3, TensorWrite<float3>>);
static_assert(std::is_same_v<Instantiable<Mul<float>>, Binary<Mul<float>>> && std::is_same_v<Instantiable<ReadU3>, Read<ReadU3>>);

// ---- data ----------------------------------------------------------------------------------------------------
static_assert(Rect(16, 32, 32, 64).x == 16 && Rect(16, 32, 32, 64).y == 32 && Rect(16, 32, 32, 64).width == 32 && Rect(16, 32, 32, 64).height == 64);
static_assert(Rect().x == 0 && Rect().height == 0 && Point().z == 0 && Size(3, 4).height == 4);
static_assert(Rect_<float, double>(1.f, 2.f, 3., 4.).width == 3.);

// ---- chains --------------------------------------------------------------------------------------------------
constexpr RawPtr<ND::_2D, uchar3> kInput{ nullptr, PtrDims<ND::_2D>(128, 64, 128 * 3) };
constexpr auto kRead = ReadU3::build(kInput);
static_assert(kRead.getActiveThreads() == ActiveThreads(128, 64, 1));

constexpr auto kCrop = kRead.then(Crop<>::build(Rect(5, 6, 30, 20)));
static_assert(std::is_same_v<std::decay_t<decltype(kCrop)>, ReadBack<Crop<Read<ReadU3>>>> && kCrop.getActiveThreads() == ActiveThreads(30, 20, 1));
static_assert(std::is_same_v<std::decay_t<decltype(Crop<Read<ReadU3>>::build(kRead, Rect(1, 1, 2, 2)))>, ReadBack<Crop<Read<ReadU3>>>>);

constexpr std::array<Rect, 2> kTwoCrops{ Rect(0, 0, 34, 25), Rect(10, 10, 70, 15) };
constexpr auto kBatchResize = kRead.then(Crop<>::build(kTwoCrops)).then(Resize<InterpolationType::INTER_LINEAR>::build(Size(100, 100)));
static_assert(kBatchResize.getActiveThreads() == ActiveThreads(100, 100, 2));
static_assert(std::decay_t<decltype(kBatchResize)>::Operation::BATCH == 2 && !isBatchOperation<std::decay_t<decltype(kCrop)>::Operation>);

// five operations fuse flat, never nested
constexpr auto kFive = kRead.then(Cast<uchar3, float3>::build())
                           .then(Mul<float3>::build(make_set<float3>(2.f)))
                           .then(Cast<float3, int3>::build())
                           .then(Cast<int3, float3>::build());
using FiveOp = std::decay_t<decltype(kFive)>::Operation;
static_assert(std::is_same_v<FiveOp, FusedOperation<ReadU3, Cast<uchar3, float3>, Mul<float3>, Cast<float3, int3>, Cast<int3, float3>>>);
static_assert(FiveOp::ParamsType::size == 5 && kFive.params.next.next.instance.params.y == 2.f, "Binary parameters reachable through next");
static_assert(sizeof(OperationTuple<Cast<int, float>, Cast<float, int>>) == 1, "Unary operations occupy no storage");
static_assert(FusedOperation<Cast<float, int>, Cast<int, float>>::exec(5.5f) == 5.f, "an all-Unary chain runs in constant expressions");
static_assert(std::is_same_v<std::decay_t<decltype(Add<int>::build(4).then(Add<int>::build(4)).then(Add<int>::build(3)))>::Operation::InstanceType, BinaryType>);
static_assert(std::decay_t<decltype(Add<int>::build(4).then(Add<int>::build(4)).then(Add<int>::build(3)))>::Operation::exec(
                  0, Add<int>::build(4).then(Add<int>::build(4)).then(Add<int>::build(3))) == 11);

// operations before a ReadBack fold into its back read; a compute operation after it gives a plain fused read
constexpr auto kCastResize = kRead.then(Cast<uchar3, float3>::build()).then(Resize<InterpolationType::INTER_LINEAR>::build(Size(16, 16)));
static_assert(isReadBackType<std::decay_t<decltype(kCastResize)>>);
static_assert(std::is_same_v<std::decay_t<decltype(kCastResize.backIOp)>::Operation, FusedOperation<ReadU3, Cast<uchar3, float3>>>);
static_assert(isReadType<std::decay_t<decltype(kCastResize.then(Mul<float3>::build(make_set<float3>(1.f))))>>);

// the README chain
constexpr std::array<Rect, 5> kReadmeCrops{ Rect(0, 0, 34, 25), Rect(10, 10, 70, 15), Rect(20, 20, 60, 59), Rect(30, 30, 20, 23), Rect(40, 40, 12, 11) };
constexpr RawPtr<ND::_2D, uchar3> k4K{ nullptr, PtrDims<ND::_2D>(3840, 2160, 3840 * 3) };
constexpr auto kReadme = ReadU3::build(k4K)
                             .then(Crop<>::build(kReadmeCrops))
                             .then(Resize<InterpolationType::INTER_LINEAR, AspectRatio::PRESERVE_AR>::build(Size(60, 60), float3{ 0.f, 0.f, 0.f }))
                             .then(Mul<float3>::build(make_set<float3>(1.4f)))
                             .then(Sub<float3>::build(make_set<float3>(0.5f)))
                             .then(Div<float3>::build(make_set<float3>(255.f)))
                             .then(ColorConversion<ColorConversionCodes::COLOR_RGB2BGR, float3, float3>::build());
using ReadmeResize = Resize<InterpolationType::INTER_LINEAR, AspectRatio::PRESERVE_AR, ReadBack<Crop<Read<ReadU3>>>>;
static_assert(std::is_same_v<std::decay_t<decltype(kReadme)>,
                             Read<BatchRead<5, PlanePolicy::PROCESS_ALL,
                                            FusedOperation<ReadmeResize, Mul<float3>, Sub<float3>, Div<float3>, VectorReorder<float3, 2, 1, 0>>>>>);
static_assert(sizeof(kReadme) == 696, "same parameter block size as the reference's README chain");
static_assert(kReadme.getActiveThreads() == ActiveThreads(60, 60, 5));
static_assert(kReadme.params.opData[3].params.instance.params.x1 == 4 && kReadme.params.opData[3].params.instance.params.x2 == 55 &&
              kReadme.params.opData[0].params.instance.params.y1 == 8 && kReadme.params.opData[0].params.instance.params.y2 == 51);

// conditional batches keep usedPlanes / default_value through then()
constexpr std::array<Size, 3> kSizes{ Size(8, 8), Size(8, 8), Size(8, 8) };
constexpr std::array<RawPtr<ND::_2D, uchar3>, 3> kThree{ kInput, kInput, kInput };
constexpr auto kCond = ReadU3::build(2, uchar3{ 1, 2, 3 }, kThree);
static_assert(std::decay_t<decltype(kCond)>::Operation::PP == PlanePolicy::CONDITIONAL_WITH_DEFAULT && kCond.params.usedPlanes == 2 && kCond.params.default_value.z == 3);
constexpr auto kCondResized = kCond.then(Resize<InterpolationType::INTER_LINEAR>::build(Size(8, 8)));
static_assert(kCondResized.params.usedPlanes == 2 && kCondResized.params.default_value.y == 2.f, "default cast to the new output type");
constexpr std::array<Read<ReadU3>, 3> kThreeReads{ kRead, kRead, kRead };
static_assert(std::decay_t<decltype(Resize<InterpolationType::INTER_LINEAR>::build(kThreeReads, kSizes))>::Operation::BATCH == 3);

// YUV front-end: a YUV read fused with its conversion is a Read that Resize accepts as its back operation, and the
// parameters of operations fused after it stay reachable (tests/operation/test_fused_operation.h:43-50 of the reference)
constexpr auto kReadYUV = ReadYUV<PixelFormat::NV12>::build({ { RawPtr<ND::_2D, uchar>{ nullptr, PtrDims<ND::_2D>(128, 128 + 64) }, 128, 128 } });
constexpr auto kReadRGB = kReadYUV.then(ConvertYUVToRGB<PixelFormat::NV12, ColorRange::Full, ColorPrimitives::bt2020, false>::build());
static_assert(isReadType<std::decay_t<decltype(kReadRGB)>> && std::is_same_v<std::decay_t<decltype(kReadRGB)>::Operation::OutputType, uchar3>);
constexpr auto kYUVResized = Resize<InterpolationType::INTER_LINEAR>::build(kReadRGB, Size(64, 64));
constexpr auto kYUVResizedDiv = kYUVResized.then(Mul<float>::build(3.f)).then(Div<float>::build(4.3f));
static_assert(kYUVResizedDiv.params.next.next.instance.params == 4.3f && kYUVResized.getActiveThreads() == ActiveThreads(64, 64, 1));
static_assert(kYUVResized.params.params.src_size.width == 128 && kYUVResized.params.src_conv_factors.x == 2.f);
// traits of the formats (raw_image.h:48-106; utest_color_conversion.h UYVY traits test of the reference)
static_assert(PixelFormatTraits<PixelFormat::UYVY>::space == ColorSpace::YUV422 && PixelFormatTraits<PixelFormat::UYVY>::depth == ColorDepth::p8bit &&
              PixelFormatTraits<PixelFormat::UYVY>::cn == 3 && PixelFormatTraits<PixelFormat::UYVY>::rf.width_f == 2.f);
static_assert(std::is_same_v<RawImage<PixelFormat::P010>::BaseType, ushort> && std::is_same_v<ReadYUV<PixelFormat::Y210>::OutputType, ushort3> &&
              std::is_same_v<YUVOutputPixelType<PixelFormat::NV21, true>, uchar4>);
static_assert(IsEven<int>::exec(4) && !IsEven<uint>::exec(7u) && IsEven<int>::exec(-2) && !IsEven<int>::exec(-1));
static_assert(ShiftRight<ushort3>::exec(ushort3{ 0xFFC0, 64, 63 }, 6).x == 1023 && ShiftLeft<ushort>::exec(1023, 6) == 0xFFC0 &&
              ShiftLeft<ushort>::exec(0xFFFF, 6) == 0xFFC0, "shifts stay in the storage type");
// studio-range grey through the bt601 matrix: (126 - 16) * 1.164383562 = 128.08 -> 128
static_assert(ConvertYUVToRGB<PixelFormat::NV12, ColorRange::Full, ColorPrimitives::bt601, true>::exec(uchar3{ 126, 128, 128 }).x == 128 &&
              ConvertYUVToRGB<PixelFormat::NV12, ColorRange::Full, ColorPrimitives::bt601, true>::exec(uchar3{ 126, 128, 128 }).w == 255);
static_assert(ConvertYUVToRGB<PixelFormat::P010, ColorRange::Full, ColorPrimitives::bt709, true>::exec(ushort3{ 500 << 6, 512 << 6, 512 << 6 }).y == (500 << 6) &&
              ConvertYUVToRGB<PixelFormat::P010, ColorRange::Full, ColorPrimitives::bt709, true>::exec(ushort3{ 500 << 6, 512 << 6, 512 << 6 }).w == (1023 << 6));
static_assert(NormalizeColorRangeDepth<float3, ColorDepth::p8bit>::exec(float3{ 0.f, 128.f, 255.f }).z == 255.f &&
              SaturateDenormalizePixel<float3, uchar3, ColorDepth::p8bit>::exec(float3{ -0.5f, 0.5f, 1.5f }).y == 127 &&
              SaturateDenormalizePixel<float3, uchar3, ColorDepth::p8bit>::exec(float3{ -0.5f, 0.5f, 1.5f }).z == 255);

// BorderReader and Warping builders (tests/algorithm/test_border_reader.h:21-30, test_warp.h:20-32 of the reference)
constexpr auto kBorder = BorderReader<BorderType::CONSTANT>::build(kRead, make_set<uchar3>(0));
static_assert(std::is_same_v<std::decay_t<decltype(kBorder)>, ReadBack<BorderReader<BorderType::CONSTANT, Read<ReadU3>>>>);
constexpr auto kWarped = kRead.then(Warping<WarpType::Perspective>::build(WarpingParameters<WarpType::Perspective>{}));
static_assert(std::is_same_v<std::decay_t<decltype(kWarped)>, ReadBack<Warping<WarpType::Perspective, Read<ReadU3>>>>);
constexpr auto kPadded = kRead.then(BorderReader<BorderType::REFLECT>::build<uchar3>()).then(Crop<>::build(Rect(static_cast<uint>(-4), static_cast<uint>(-4), 72, 40)));
static_assert(kPadded.getActiveThreads() == ActiveThreads(72, 40, 1) && std::is_same_v<std::decay_t<decltype(kPadded)>::Operation::OutputType, uchar3>);
static_assert(kRead.then(BorderReader<BorderType::CONSTANT>::build(uchar3{ 1, 2, 3 })).params.value.z == 3);
static_assert(detail::border_index<BorderType::REFLECT>(-6, 8) == 5 && detail::border_index<BorderType::REFLECT>(14, 8) == 1 &&
              detail::border_index<BorderType::REFLECT_101>(-6, 8) == 6 && detail::border_index<BorderType::REFLECT_101>(14, 8) == 0 &&
              detail::border_index<BorderType::WRAP>(-6, 8) == 2 && detail::border_index<BorderType::WRAP>(14, 8) == 6 &&
              detail::border_index<BorderType::REPLICATE>(-6, 8) == 0 && detail::border_index<BorderType::REPLICATE>(14, 8) == 7,
              "the border diagrams of border_reader.h:26-33");
static_assert(sizeof(WarpingParameters<WarpType::Affine>) == 32 && sizeof(WarpingParameters<WarpType::Perspective>) == 44);

// StaticLoop (algorithms/basic_ops/static_loop.h:21-45 of the reference): N applications, at least one
static_assert(StaticLoop<Add<int>, 5>::exec(1, 2) == 11 && StaticLoop<Add<int>, 1>::exec(1, 2) == 3 && StaticLoop<Add<int>, 0>::exec(1, 2) == 3);
static_assert(StaticLoop<StaticLoop<Mul<int>, 3>, 2>::exec(1, 2) == 64 && isBinaryType<StaticLoop<Add<float>, 4>>);

// circular memory operations and CircularTensor (memory_operations.h:425-443, circular_tensor.h:24-61 of the reference)
static_assert(circular_batch_internal::computeCircularThreadIdx<CircularDirection::Ascendent, 4>(Point(1, 2, 3), 2).z == 1 &&
              circular_batch_internal::computeCircularThreadIdx<CircularDirection::Descendent, 4>(Point(1, 2, 3), 2).z == 3 &&
              circular_batch_internal::computeCircularThreadIdx<CircularDirection::Descendent, 4>(Point(1, 2, 1), 2).z == 1);
static_assert(SequenceSelectorType<CircularTensorOrder::NewestFirst, 4>::at(0) == 1 && SequenceSelectorType<CircularTensorOrder::NewestFirst, 4>::at(3) == 2 &&
              SequenceSelectorType<CircularTensorOrder::OldestFirst, 4>::at(3) == 1 && SequenceSelectorType<CircularTensorOrder::OldestFirst, 4>::at(0) == 2);
static_assert(CTReadDirection_v<CircularTensorOrder::NewestFirst> == CircularDirection::Descendent &&
              std::is_same_v<CircularTensorStoreType<float, 3>::type, float3> && std::is_same_v<CircularTensorStoreType<uchar4, 1>::type, uchar4> &&
              std::is_base_of_v<TensorT<float>, CircularTensor<float, 3, 4, CircularTensorOrder::OldestFirst, ColorPlanes::Transposed>>);
static_assert(isWriteType<Write<TensorTSplit<float3>>> && isReadType<Read<TensorPack<float3>>> && isReadType<Read<TensorTPack<uchar4>>> &&
              isReadType<Read<CircularTensorRead<CircularDirection::Ascendent, TensorRead<float3>, 4>>> &&
              isWriteType<Write<CircularBatchWrite<CircularDirection::Ascendent, PerThreadWrite<ND::_2D, float>, 4>>>);

// known answers of the reference's unit tests for single operations (utests/algorithm/image_processing/
// utest_color_conversion.h:34-224; where its harness compares one channel, x, the values of that channel)
static_assert(IsEven<uint>::exec(0u) && !IsEven<uint>::exec(1u) && IsEven<uint>::exec(2u) && !IsEven<uint>::exec(3u));
static_assert(AddOpaqueAlpha<uchar3, ColorDepth::p8bit>::exec(uchar3{ 100, 150, 200 }).w == 255 && AddOpaqueAlpha<uchar3, ColorDepth::p8bit>::exec(uchar3{ 50, 75, 125 }).x == 50 &&
              StaticAddAlpha<uchar3, 255>::exec(uchar3{ 100, 150, 200 }).w == 255 && StaticAddAlpha<uchar3, 7>::exec(uchar3{ 50, 75, 125 }).w == 7);
static_assert(ColorConversion<ColorConversionCodes::COLOR_BGR2BGRA, uchar3, uchar4>::exec(uchar3{ 100, 150, 200 }).z == 200 &&
              ColorConversion<ColorConversionCodes::COLOR_BGR2BGRA, uchar3, uchar4>::exec(uchar3{ 100, 150, 200 }).w == 255 &&
              ColorConversion<ColorConversionCodes::COLOR_BGR2RGB, uchar3, uchar3>::exec(uchar3{ 100, 150, 200 }).x == 200 &&
              ColorConversion<ColorConversionCodes::COLOR_BGR2RGB, uchar3, uchar3>::exec(uchar3{ 50, 75, 125 }).z == 50);
static_assert(DenormalizePixel<float3, ColorDepth::p8bit>::exec(float3{ 0.0f, 0.5f, 1.0f }).y == 127.5f && DenormalizePixel<float3, ColorDepth::p8bit>::exec(float3{ 0.25f, 0.75f, 0.9f }).x == 63.75f &&
              NormalizePixel<uchar3, ColorDepth::p8bit>::exec(uchar3{ 0, 128, 255 }).z == 1.0f && NormalizePixel<uchar3, ColorDepth::p8bit>::exec(uchar3{ 64, 192, 32 }).x == 64.0f / 255.0f &&
              SaturateDenormalizePixel<float3, uchar3, ColorDepth::p8bit>::exec(float3{ -0.5f, 0.5f, 1.5f }).x == 0 &&
              SaturateDenormalizePixel<float3, uchar3, ColorDepth::p8bit>::exec(float3{ 0.25f, 0.75f, 0.9f }).x == 63 &&
              NormalizeColorRangeDepth<float3, ColorDepth::p8bit>::exec(float3{ 64.0f, 192.0f, 100.0f }).y == 192.0f);
// Deinterlace builders (tests/algorithm/test_deinterlace.h:21-44 of the reference)
constexpr auto kBlend = Deinterlace<DeinterlaceType::BLEND>::build(kRead);
constexpr auto kLinear = Deinterlace<DeinterlaceType::INTER_LINEAR>::build(DeinterlaceLinear::USE_EVEN, kRead);
static_assert(std::is_same_v<std::decay_t<decltype(kBlend)>, ReadBack<Deinterlace<DeinterlaceType::BLEND, Read<ReadU3>>>> &&
              std::is_same_v<std::decay_t<decltype(kLinear)>, ReadBack<Deinterlace<DeinterlaceType::INTER_LINEAR, Read<ReadU3>>>> && kLinear.params.useEvenLines &&
              std::is_same_v<std::decay_t<decltype(kRead.then(Deinterlace<DeinterlaceType::BLEND>::build()))>, std::decay_t<decltype(kBlend)>> &&
              std::is_same_v<std::decay_t<decltype(kBlend)>::Operation::OutputType, float3>);

// SaturateCast over every pair of base types, at the lowest, half the highest and the highest input: the expectations
// of the reference's utests/algorithm/image_processing/utest_saturate.h:46-85 (clamped to the output range, otherwise
// the plain cast)
template <typename I, typename O>
constexpr bool saturate_pair_ok() {
    constexpr I lowest = minValue<I>, half = maxValue<I> / 2, highest = maxValue<I>;
    constexpr O want_low = cxp::cmp_less(lowest, minValue<O>) || !cxp::cmp_greater(lowest, minValue<O>) ? minValue<O> : static_cast<O>(lowest);
    constexpr O want_half = cxp::cmp_greater(half, maxValue<O>) ? maxValue<O> : static_cast<O>(half);
    constexpr O want_high = cxp::cmp_greater(highest, maxValue<O>) ? maxValue<O> : static_cast<O>(highest);
    return SaturateCast<I, O>::exec(lowest) == want_low && SaturateCast<I, O>::exec(half) == want_half && SaturateCast<I, O>::exec(highest) == want_high &&
           SaturateCast<VectorType_t<I, 3>, VectorType_t<O, 3>>::exec(make_set<VectorType_t<I, 3>>(highest)).z == want_high &&
           SaturateCast<VectorType_t<I, 4>, VectorType_t<O, 4>>::exec(make_set<VectorType_t<I, 4>>(lowest)).w == want_low;
}
template <typename I, typename... Os>
constexpr bool saturate_row_ok(TypeList<Os...>) {
    return (saturate_pair_ok<I, Os>() && ...);
}
template <typename... Is>
constexpr bool saturate_table_ok(TypeList<Is...> all) {
    return (saturate_row_ok<Is>(all) && ...);
}
// integer -> float pairs are exact only while the integer fits the mantissa, so half / highest of 32-bit integers go
// through the same cast on both sides and still compare equal
static_assert(saturate_table_ok(TypeList<unsigned char, signed char, unsigned short, short, unsigned int, int, float, double>{}));
static_assert(SaturateCast<float, uchar>::exec(254.5f) == 255 && SaturateCast<float, uchar>::exec(254.49f) == 254 && SaturateCast<float, uchar>::exec(0.5f) == 1 &&
              SaturateCast<float, uchar>::exec(0.49999997f) == 1 && SaturateCast<float, uchar>::exec(0.4999999f) == 0 && SaturateCast<float, signed char>::exec(-0.5f) == -1 &&
              SaturateCast<float, signed char>::exec(-128.7f) == -128 && SaturateCast<float, short>::exec(-2.5f) == -3 && SaturateCast<double, ushort>::exec(65534.5) == 65535,
              "half away from zero through x + 0.5f (so the float just below one half rounds up, as in the reference), then the range");

// DPP tags
static_assert(TransformDPP<>::PAR_ARCH == ParArch::GPU_AMD && defaultParArch == ParArch::GPU_AMD && Stream::parArch() == ParArch::GPU_AMD);
static_assert(exec::pixels_per_thread<float3, float3, false>() == 4 && exec::pixels_per_thread<uchar4, uchar, false>() == 4 &&
              exec::pixels_per_thread<uchar4, float3, false>() == 4 && exec::pixels_per_thread<uchar, uchar, false>() == 16);

// Every public name of the reference's namespace fk (tests/golden/reference_public_names.txt, listed from its headers by
// tests/golden/make_reference_names.py) exists in this library's fk: a using-declaration of a name that is missing does not
// compile.  The names that are deliberately absent, each with its reason, are in tests/golden/reference_names_absent.txt.
namespace reference_names {
#define FK_REFERENCE_NAME(name) using fk::name;
#include "reference_names.inc"
#undef FK_REFERENCE_NAME
} // namespace reference_names

int main() {
    int failures = 0;
    // RGB2Gray known answers of the reference's unit test (rounding to nearest is not a constant expression)
    EXPECT((RGB2Gray<uchar3, uchar>::exec(uchar3{ 255, 0, 0 }) == 76 && RGB2Gray<uchar3, uchar>::exec(uchar3{ 0, 255, 0 }) == 150 &&
            RGB2Gray<uchar3, uchar>::exec(uchar3{ 0, 0, 255 }) == 29));
    EXPECT((RGB2Gray<uchar3, uchar, GrayFormula::CCIR_601>::exec(uchar3{ 50, 100, 150 }) == 91 &&
            RGB2Gray<uchar3, uchar, GrayFormula::CCIR_601>::exec(uchar3{ 75, 125, 200 }) == 119));
    // owning host buffers: refcount through copies, crop views share ownership, at() addresses by pitch
    {
        Ptr2D<uchar3> img(64, 32, 0, MemType::Host);
        EXPECT(img.getRefCount() == 1 && img.dims().pitch == 64 * 3 && img.sizeInBytes() == 64u * 32u * 3u);
        {
            Ptr2D<uchar3> copy = img;
            EXPECT(img.getRefCount() == 2);
            auto view = copy.crop2D(Point(4, 2), PtrDims<ND::_2D>(8, 8));
            EXPECT(img.getRefCount() == 3 && view.dims().pitch == img.dims().pitch);
            img.at(4, 2) = uchar3{ 9, 8, 7 };
            EXPECT(view.at(0, 0).x == 9 && view.at(0, 0).z == 7);
        }
        EXPECT(img.getRefCount() == 1);
        Tensor<float3> t(6, 5, 4, 1, MemType::Host);
        EXPECT(t.dims().pitch == 6 * sizeof(float3) && t.dims().plane_pitch == 6 * 5 * sizeof(float3) && t.getNumElements() == 120);
        t.at(1, 2, 3) = float3{ 1.f, 2.f, 3.f };
        auto plane = t.getPlane(3);
        EXPECT(plane.at(1, 2).y == 2.f && t.getRefCount() == 2);
    }
    // misuse throws, as the reference's Ptr does
    {
        bool threw = false;
        try {
            uchar3 pixel{};
            Ptr2D<uchar3> bad(&pixel, 1, 1, 3, MemType::DeviceAndPinned);
        } catch (const std::runtime_error&) {
            threw = true;
        }
        EXPECT(threw);
        threw = false;
        try {
            Ptr2D<uchar3> host(4, 4, 0, MemType::Host), other(4, 4, 0, MemType::Host);
            host.uploadTo(other); // destination is not device memory
        } catch (const std::runtime_error&) {
            threw = true;
        }
        EXPECT(threw);
        threw = false;
        try {
            Ptr2D<uchar3> twice(4, 4, 0, MemType::Host);
            twice.Alloc(Size(4, 4), 0, MemType::Host);
        } catch (const std::runtime_error&) {
            threw = true;
        }
        EXPECT(threw);
    }
    // host evaluation of a chain element by element (the operations are plain host+device functions)
    {
        Ptr2D<uchar3> img(16, 16, 0, MemType::Host);
        for (uint y = 0; y < 16; ++y)
            for (uint x = 0; x < 16; ++x) img.at(x, y) = uchar3{ static_cast<uchar>(x), static_cast<uchar>(y), 5 };
        const auto chain = PerThreadRead<ND::_2D, uchar3>::build(img.ptrPinned())
                               .then(Crop<>::build(Rect(2, 3, 8, 8)))
                               .then(Resize<InterpolationType::INTER_LINEAR>::build(Size(8, 8)))
                               .then(ColorConversion<ColorConversionCodes::COLOR_RGB2BGR, float3, float3>::build());
        const float3 v = std::decay_t<decltype(chain)>::Operation::exec(Point(1, 2), chain);
        EXPECT(v.x == 5.f && v.y == 5.f && v.z == 3.f); // identity resize of the crop, channels reversed
        const auto view = exec::ViewOf<std::decay_t<decltype(PerThreadRead<ND::_2D, uchar3>::build(img.ptrPinned()).then(Crop<>::build(Rect(2, 3, 8, 8))))>>::make(
            PerThreadRead<ND::_2D, uchar3>::build(img.ptrPinned()).then(Crop<>::build(Rect(2, 3, 8, 8))));
        EXPECT(view.ox == 2 && view.oy == 3 && view.w == 8 && view.h == 8 && view.img_w == 16);
    }
    if (failures == 0) std::printf("conformance ok\n");
    return failures == 0 ? 0 : 1;
}
