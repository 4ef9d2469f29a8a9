// Names of the reference's namespace fk that user code may spell and that this library has under another spelling or did
// not need for itself: the struct forms behind the `_t` / `_v` aliases, the capitalised names of the vector structs, the
// member-detection traits of the operation model, and a few small operations and holders.
//
// Counterpart of (reference, include/fused_kernel/): core/data/vector_types.h:68-262 (struct names of the vector types),
// core/utils/type_lists.h:154-255 (TypeAt, EquivalentType, InsertType, RemoveType, all_types_are_same),
// core/execution_model/operation_model/operation_data.h:22-77 (hasParams, has_next, hasBackIOp ...),
// operation_types.h:30-185 (HasInstanceType, NotAllUnary, are_all_unary_types, IsCompleteOperation, is_fused_operation_),
// batch_operations.h:22-40,213-216 (has_batch, has_operation, IsBatchOperation, NullTypeToUchar, NullTypeToAlternative),
// operation_tuple.h:127-205 (OperationTupleTypeToTypeList, TypeListToOperationTuple, get_ot, HasOperation,
// IsInstantiableOperation), fused_operation.h:119-133,337-341 (FusedOperationOutputType, FOOT,
// IsNotAllUnaryFusedOperation), core/data/tuple.h:139-147,243-259 (TupleTypeToTypeList, GetFirst, GetSecond),
// core/utils/cuda_vector_utils.h:232-290 (make, UnaryVectorSet), core/data/rawptr.h:241-294 (StaticPtrAccessor, StaticPtr),
// algorithms/basic_ops/cast_base.h:19-32 (CastBase), algorithms/basic_ops/logical.h:25-43 (ShiftBase),
// algorithms/image_processing/saturate.h:68-93 (SaturateFloatBase, Saturate), interpolation.h:25-31 (Slice2x2),
// resize.h:26-41 (ComputeResizePoint), raw_image.h:24-35 (CS_t, CD_t and the depth lists),
// color_conversion.h:26-27,535-549 (VOneMore, CCC_t, SupportedCCC, isSuportedCCC),
// core/execution_model/thread_fusion.h:50-58 (TFSourceTypes, TFBiggerTypes, FilteredType_t).
#ifndef FK_CORE_REFERENCE_SURFACE_H
#define FK_CORE_REFERENCE_SURFACE_H

#include "fk/ops/image_processing.h"
#include "fk/ops/yuv.h"

namespace fk {

// ---- the vector structs under their struct names (the lower-case names are the ones everything else uses) ----------
#define FK_VECTOR_STRUCT_NAMES(Upper, lower) \
    using Upper##1 = lower##1;               \
    using Upper##2 = lower##2;               \
    using Upper##3 = lower##3;               \
    using Upper##4 = lower##4;
FK_VECTOR_STRUCT_NAMES(Char, char)
FK_VECTOR_STRUCT_NAMES(Uchar, uchar)
FK_VECTOR_STRUCT_NAMES(Short, short)
FK_VECTOR_STRUCT_NAMES(Ushort, ushort)
FK_VECTOR_STRUCT_NAMES(Int, int)
FK_VECTOR_STRUCT_NAMES(Uint, uint)
FK_VECTOR_STRUCT_NAMES(Long, long)
FK_VECTOR_STRUCT_NAMES(Ulong, ulong)
FK_VECTOR_STRUCT_NAMES(Longlong, longlong)
FK_VECTOR_STRUCT_NAMES(Ulonglong, ulonglong)
FK_VECTOR_STRUCT_NAMES(Float, float)
FK_VECTOR_STRUCT_NAMES(Double, double)
#undef FK_VECTOR_STRUCT_NAMES

// ---- type lists: the struct forms ------------------------------------------------------------------------------------
template <int N, typename List>
struct TypeAt {
    using type = TypeAt_t<N, List>;
};
template <typename T, typename ListOne, typename ListTwo>
struct EquivalentType {
    static_assert(one_of_v<T, ListOne>, "The type is not in the first list");
    using type = EquivalentType_t<T, ListOne, ListTwo>;
};
template <size_t N, typename T, typename List = TypeList<>>
struct InsertType {
    using type = InsertType_t<N, T, List>;
};
template <size_t N, typename List>
struct RemoveType {
    using type = RemoveType_t<N, List>;
};
template <typename T, typename... Ts>
constexpr bool all_types_are_same = (std::is_same_v<T, Ts> && ...);

// ---- member detection on operations and instantiable operations ---------------------------------------------------
template <typename T, typename = void>
struct hasParams : std::false_type {};
template <typename T>
struct hasParams<T, std::void_t<typename T::ParamsType>> : std::true_type {};
template <typename T>
constexpr bool hasParams_v = hasParams<T>::value;

template <typename T, typename = void>
struct has_next : std::false_type {};
template <typename T>
struct has_next<T, std::void_t<decltype(std::declval<T>().next)>> : std::true_type {};
template <typename T>
constexpr bool has_next_v = has_next<T>::value;

using BFList = TypeList<ReadBackType, TernaryType>; // the kinds that carry a back operation
template <typename OpOrIOp>
constexpr bool hasNoBackIOp_v = !one_of_v<typename OpOrIOp::InstanceType, BFList>;

template <typename T, typename = void>
struct hasBackIOp : std::false_type {};
template <typename T>
struct hasBackIOp<T, std::void_t<typename T::BackIOp>> : std::true_type {};
template <typename T>
constexpr bool hasBackIOp_v = hasBackIOp<T>::value;

template <typename T, typename = void>
struct hasParamsAndBackIOp : std::false_type {};
template <typename T>
struct hasParamsAndBackIOp<T, std::void_t<typename T::ParamsType, typename T::BackIOp>> : std::true_type {};
template <typename T>
constexpr bool hasParamsAndBackIOp_v = hasParamsAndBackIOp<T>::value;

namespace detail {
template <typename Operation, bool = hasParams_v<Operation>>
struct ParamsAreArray : std::false_type {};
template <typename Operation>
struct ParamsAreArray<Operation, true> : std::is_array<typename Operation::ParamsType> {};
} // namespace detail
template <typename Operation>
constexpr bool hasParamsNoArray = hasParams_v<Operation> && !detail::ParamsAreArray<Operation>::value;
template <typename Operation>
constexpr bool hasParamsArray = detail::ParamsAreArray<Operation>::value;

template <typename T, typename = void>
struct HasInstanceType : std::false_type {};
template <typename T>
struct HasInstanceType<T, std::void_t<typename T::InstanceType>> : std::true_type {};

template <typename Enabler = void, typename... OpsOrIOps>
struct NotAllUnary final : std::bool_constant<((!std::is_same_v<typename OpsOrIOps::InstanceType, UnaryType>) || ...)> {};
template <typename Enabler, typename... OpsOrIOps>
struct are_all_unary_types : std::bool_constant<(sizeof...(OpsOrIOps) > 0) && (std::is_same_v<typename OpsOrIOps::InstanceType, UnaryType> && ...)> {};

template <typename T, typename = void>
struct IsCompleteOperation : std::false_type {};
template <typename T>
struct IsCompleteOperation<T, std::void_t<decltype(&T::exec)>> : std::true_type {};

namespace detail {
template <typename T, typename = void>
struct DeclaresFusedOp : std::false_type {};
template <typename T>
struct DeclaresFusedOp<T, std::void_t<decltype(T::IS_FUSED_OP)>> : std::bool_constant<T::IS_FUSED_OP> {};
} // namespace detail
template <typename Enabler, typename T>
struct is_fused_operation_ : detail::DeclaresFusedOp<T> {};

template <typename T, typename = void>
struct has_batch : std::false_type {};
template <typename T>
struct has_batch<T, std::void_t<decltype(T::BATCH)>> : std::is_integral<std::decay_t<decltype(T::BATCH)>> {};
template <typename T, typename = void>
struct has_operation : std::false_type {};
template <typename T>
struct has_operation<T, std::void_t<typename T::Operation>> : std::true_type {};
template <typename T>
struct IsBatchOperation : std::bool_constant<has_batch<T>::value && has_operation<T>::value> {};

template <typename T>
using NullTypeToUchar = std::conditional_t<std::is_same_v<T, NullType>, uchar, T>;
template <typename Nullable, typename Alternative>
using NullTypeToAlternative = std::conditional_t<std::is_same_v<Nullable, NullType>, Alternative, Nullable>;

template <typename Type, typename = void>
struct HasOperation : std::false_type {};
template <typename Type>
struct HasOperation<Type, std::void_t<typename Type::Operation>> : std::true_type {};
// a restriction for filtered_index_sequence_t: the entries that are instantiable operations
struct IsInstantiableOperation {
    template <typename Type>
    FK_HD_STATIC bool complies() { return HasOperation<Type>::value; }
};

// the instantiable form of an operation, as a struct (instantiable_operations.h:177-212)
template <typename Operation, typename Enabler = void>
struct InstantiableOperationType {
    using type = Instantiable<Operation>;
};

// ---- tuples and operation tuples as type lists -------------------------------------------------------------------------
template <typename TupleType>
struct TupleTypeToTypeList;
template <typename... Types>
struct TupleTypeToTypeList<Tuple<Types...>> {
    using type = TypeList<Types...>;
};
template <typename TupleType>
struct OperationTupleTypeToTypeList;
template <typename... Operations>
struct OperationTupleTypeToTypeList<OperationTuple<Operations...>> {
    using type = TypeList<Operations...>;
};
template <typename TupleType>
using OTToTypeList = typename OperationTupleTypeToTypeList<TupleType>::type;
template <typename List>
struct TypeListToOperationTuple;
template <typename... Operations>
struct TypeListToOperationTuple<TypeList<Operations...>> {
    using type = OperationTuple<Operations...>;
};
template <typename List>
using TypeListToOT = typename TypeListToOperationTuple<List>::type;
template <int INDEX, typename TupleType>
using get_ot = TypeAt_t<INDEX, OTToTypeList<TupleType>>;
template <int INDEX, typename TupleType>
struct GetType {
    using type = get_ot<INDEX, TupleType>;
};

// what a fused operation yields when its last operation is this one: a write passes its input on
template <typename Enabler, typename... Operations>
struct FusedOperationOutputType;
template <typename Operation>
struct FusedOperationOutputType<std::enable_if_t<isWriteType<Operation>>, Operation> {
    using type = typename Operation::InputType;
};
template <typename Operation>
struct FusedOperationOutputType<std::enable_if_t<!isWriteType<Operation>>, Operation> {
    using type = typename Operation::OutputType;
};
template <typename... Operations>
using FOOT = typename FusedOperationOutputType<void, Operations...>::type;
// a fused operation of unary operations only exposes its list of operations
template <typename FusedOperationType, typename = void>
struct IsNotAllUnaryFusedOperation : std::true_type {};
template <typename FusedOperationType>
struct IsNotAllUnaryFusedOperation<FusedOperationType, std::void_t<typename FusedOperationType::Operations>> : std::false_type {};

// element selectors of a pair, in the form that the batch builders' translate step takes
template <typename FirstType, typename SecondType>
struct GetFirst {
    using OutputType = FirstType;
    template <int Idx>
    static constexpr FirstType translate(const int&, const std::pair<FirstType, SecondType>& p) { return p.first; }
};
template <typename FirstType, typename SecondType>
struct GetSecond {
    using OutputType = SecondType;
    template <int Idx>
    static constexpr SecondType translate(const int&, const std::pair<FirstType, SecondType>& p) { return p.second; }
};

// ---- building vector values -------------------------------------------------------------------------------------------------
struct make {
    template <typename T, typename... Numbers>
    FK_HD_STATIC T type(const Numbers&... pack) {
        static_assert(validCUDAVec<T>, "make::type<T>: T is not a vector type");
        static_assert(sizeof...(Numbers) == cn<T>, "make::type<T>: one value per channel");
        return T{ static_cast<VBase<T>>(pack)... };
    }
};
template <typename T, typename Enabler = void>
struct UnaryVectorSet {
    FK_HD_STATIC T exec(const T& value) { return value; }
};
template <typename T>
struct UnaryVectorSet<T, std::enable_if_t<validCUDAVec<T>>> {
    FK_HD_STATIC T exec(const VBase<T>& value) { return make_set<T>(value); }
};

// ---- static pointers ----------------------------------------------------------------------------------------------------------
template <ND D>
struct StaticPtrAccessor;
template <>
struct StaticPtrAccessor<ND::_1D> {
    template <int W, typename T>
    FK_HD_STATIC T read(const Point& p, const StaticRawPtr<StaticPtrDims1D<W>, T>& ptr) { return ptr.data[p.x]; }
    template <int W, typename T>
    FK_HD_STATIC void write(const Point& p, StaticRawPtr<StaticPtrDims1D<W>, T>& ptr, const T& value) { ptr.data[p.x] = value; }
};
template <>
struct StaticPtrAccessor<ND::_2D> {
    template <int W, int H, typename T>
    FK_HD_STATIC T read(const Point& p, const StaticRawPtr<StaticPtrDims2D<W, H>, T>& ptr) { return ptr.data[p.y][p.x]; }
    template <int W, int H, typename T>
    FK_HD_STATIC void write(const Point& p, StaticRawPtr<StaticPtrDims2D<W, H>, T>& ptr, const T& value) { ptr.data[p.y][p.x] = value; }
};
template <>
struct StaticPtrAccessor<ND::_3D> {
    template <int W, int H, int P, typename T>
    FK_HD_STATIC T read(const Point& p, const StaticRawPtr<StaticPtrDims3D<W, H, P>, T>& ptr) { return ptr.data[p.z][p.y][p.x]; }
    template <int W, int H, int P, typename T>
    FK_HD_STATIC void write(const Point& p, StaticRawPtr<StaticPtrDims3D<W, H, P>, T>& ptr, const T& value) { ptr.data[p.z][p.y][p.x] = value; }
};
template <typename StaticRawPtrType>
struct StaticPtr {
    using Type = typename StaticRawPtrType::type;
    using At = StaticPtrAccessor<static_cast<ND>(StaticRawPtrType::NDim)>;
    StaticRawPtrType ptr_a;
    constexpr StaticRawPtrType ptr() const { return ptr_a; }
    constexpr auto dims() const { return ptr_a.dims; }
};

// ---- small operations ------------------------------------------------------------------------------------------------------------
// static_cast of a scalar
template <typename I, typename O>
struct CastBase {
private:
    using SelfType = CastBase<I, O>;

public:
    FK_UNARY_OPERATION(CastBase, I, O)
    FK_HD_STATIC OutputType exec(const InputType& input) { return static_cast<O>(input); }
};
// shift of an unsigned scalar
template <typename T, ShiftDirection SD>
struct ShiftBase {
private:
    using SelfType = ShiftBase<T, SD>;

public:
    FK_BINARY_OPERATION(ShiftBase, T, uint, T)
    static_assert(!validCUDAVec<T>, "ShiftBase takes scalars; Shift takes vectors");
    static_assert(std::is_unsigned_v<T>, "Shift only works with unsigned integers.");
    FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) {
        if constexpr (SD == ShiftDirection::Left) return static_cast<T>(input << params);
        else return static_cast<T>(input >> params);
    }
};
// a float clamped to [0, 1]
struct SaturateFloatBase {
private:
    using SelfType = SaturateFloatBase;

public:
    FK_UNARY_OPERATION(SaturateFloatBase, float, float)
    FK_HD_STATIC OutputType exec(const InputType& input) { return detail::clamp_float(input, 0.f, 1.f); }
};
// a scalar clamped to [params.x, params.y]
template <typename T>
struct Saturate {
private:
    using SelfType = Saturate<T>;
    using Limits = VectorType_t<VBase<T>, 2>;

public:
    FK_BINARY_OPERATION(Saturate, T, Limits, T)
    static_assert(!validCUDAVec<T>, "Saturate only works with non vector types");
    FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) {
        const T capped = input < params.y ? input : params.y; // min(input, high), then max(.., low)
        return capped > params.x ? capped : params.x;
    }
};
// the source position of a destination pixel under a resize: (x * fx, y * fy)
struct ComputeResizePoint {
private:
    using SelfType = ComputeResizePoint;

public:
    FK_BINARY_OPERATION(ComputeResizePoint, Point, float2, float2)
    FK_HD_STATIC OutputType exec(const InputType& thread, const ParamsType& params) {
        return float2{ static_cast<float>(thread.x) * params.x, static_cast<float>(thread.y) * params.y };
    }
};
// the 2x2 neighbourhood of an interpolation
template <typename T>
struct Slice2x2 {
    T _0x0;
    T _1x0;
    T _0x1;
    T _1x1;
};

// ---- enum values as types, and the lists built from them ---------------------------------------------------------------------
template <ColorSpace CS>
struct CS_t {
    ColorSpace value{ CS };
};
template <ColorDepth CD>
struct CD_t {
    ColorDepth value{ CD };
};
using ColorDepthTypes = TypeList<CD_t<ColorDepth::p8bit>, CD_t<ColorDepth::p10bit>, CD_t<ColorDepth::p12bit>, CD_t<ColorDepth::f24bit>>;
using ColorDepthPixelBaseTypes = TypeList<ColorDepthPixelBaseType<ColorDepth::p8bit>, ColorDepthPixelBaseType<ColorDepth::p10bit>,
                                          ColorDepthPixelBaseType<ColorDepth::p12bit>, ColorDepthPixelBaseType<ColorDepth::f24bit>>;
using ColorDepthPixelTypes = TypeList<ColorDepthPixelType<ColorDepth::p8bit>, ColorDepthPixelType<ColorDepth::p10bit>,
                                      ColorDepthPixelType<ColorDepth::p12bit>, ColorDepthPixelType<ColorDepth::f24bit>>;

template <typename I>
using VOneMore = VectorType_t<VBase<I>, cn<I> + 1>;
template <ColorConversionCodes value>
using CCC_t = E_t<ColorConversionCodes, value>;
using SupportedCCC =
    TypeList<CCC_t<ColorConversionCodes::COLOR_BGR2BGRA>, CCC_t<ColorConversionCodes::COLOR_RGB2RGBA>, CCC_t<ColorConversionCodes::COLOR_BGRA2BGR>,
             CCC_t<ColorConversionCodes::COLOR_RGBA2RGB>, CCC_t<ColorConversionCodes::COLOR_BGR2RGBA>, CCC_t<ColorConversionCodes::COLOR_RGB2BGRA>,
             CCC_t<ColorConversionCodes::COLOR_BGRA2RGB>, CCC_t<ColorConversionCodes::COLOR_RGBA2BGR>, CCC_t<ColorConversionCodes::COLOR_BGR2RGB>,
             CCC_t<ColorConversionCodes::COLOR_RGB2BGR>, CCC_t<ColorConversionCodes::COLOR_BGRA2RGBA>, CCC_t<ColorConversionCodes::COLOR_RGBA2BGRA>,
             CCC_t<ColorConversionCodes::COLOR_RGB2GRAY>, CCC_t<ColorConversionCodes::COLOR_RGBA2GRAY>, CCC_t<ColorConversionCodes::COLOR_BGR2GRAY>,
             CCC_t<ColorConversionCodes::COLOR_BGRA2GRAY>>;
template <ColorConversionCodes CODE>
constexpr bool isSuportedCCC = one_of_v<CCC_t<CODE>, SupportedCCC>;
using detail::ColorConversionType;

// ---- thread fusion: the type that holds two (or four) elements of a source type ------------------------------------------
using TFSourceTypes = TypeListCat_t<BaseTypes, VOne, VTwo, VThree, VFour>;
using TFBiggerTypes = TypeList<bool4, uchar4, char4, ushort2, short2, uint2, int2, ulong, long, ulonglong, longlong, float2, double,
                               bool4, uchar4, char4, ushort2, short2, uint2, int2, ulong, long, ulonglong, longlong, float2, double,
                               bool4, uchar4, char4, ushort2, short2, uint2, int2, ulong2, long2, ulonglong2, longlong2, float2, double2,
                               bool3, uchar3, char3, ushort3, short3, uint3, int3, ulong3, long3, ulonglong3, longlong3, float3, double3,
                               bool4, uchar4, char4, ushort4, short4, uint4, int4, ulong4, long4, ulonglong4, longlong4, float4, double4>;
template <typename T>
using FilteredType_t = std::conditional_t<std::is_same_v<T, char>, VBase<T>, T>;

} // namespace fk
#endif
