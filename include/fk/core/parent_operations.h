// The building blocks user code defines its own operations with, in the style of the Fused Kernel Library:
//
//     template <typename T>
//     struct Twice {
//     private:
//         using SelfType = Twice<T>;
//     public:
//         FK_STATIC_STRUCT(Twice, SelfType)
//         using Parent = UnaryOperation<T, T, Twice<T>>;
//         DECLARE_UNARY_PARENT
//         FK_HOST_DEVICE_FUSE OutputType exec(const InputType& input) { return input + input; }
//     };
//
// A parent names the member types of one kind of operation (and the build() / exec(opData) forms that follow from them);
// the DECLARE_*_PARENT macro of that kind imports them into the operation.  Same parents, template parameters and macro
// names as the reference's core/execution_model/operation_model/parent_operations.h:23-281 and the batch halves of its
// read / write parents (batch_operations.h:408-450).  The operations of this library spell their members out directly,
// so these exist for operations written against the reference.
#ifndef FK_CORE_PARENT_OPERATIONS_H
#define FK_CORE_PARENT_OPERATIONS_H

#include "fk/core/operation_model.h"
#include "fk/core/thread_fusion_info.h"

namespace fk {
namespace detail {
// What every parent has: the kind, the instantiable form of the child and the fused flag.  OperationData<Child> is named
// with its kind spelled out, because inside a parent the child is still incomplete and cannot be asked for its kind.
template <typename Kind, typename Child_, bool IS_FUSED>
struct ParentCommon {
    using Child = Child_;
    using InstanceType = Kind;
    using InstantiableType = typename InstantiableFor<Child_, Kind>::type;
    using OperationDataType = OperationData<Child_, Kind>;
    static constexpr bool IS_FUSED_OP = IS_FUSED;
};
// build() forms shared by the kinds that carry parameters only / parameters and a back operation
template <typename Common, typename Params>
struct BuildFromParams {
    FK_HD_STATIC typename Common::InstantiableType build(const typename Common::OperationDataType& opData) {
        return typename Common::InstantiableType{ opData };
    }
    FK_HD_STATIC typename Common::InstantiableType build(const Params& params) { return typename Common::InstantiableType{ { params } }; }
};
template <typename Common, typename Params, typename Back>
struct BuildFromParamsAndBack {
    FK_HD_STATIC typename Common::InstantiableType build(const typename Common::OperationDataType& opData) {
        return typename Common::InstantiableType{ opData };
    }
    FK_HD_STATIC typename Common::InstantiableType build(const Params& params, const Back& backIOp) {
        return typename Common::InstantiableType{ { params, backIOp } };
    }
};
} // namespace detail

template <typename I, typename O, typename Child, bool IS_FUSED = false>
struct UnaryOperation : detail::ParentCommon<UnaryType, Child, IS_FUSED> {
    using InputType = I;
    using OutputType = O;
    FK_HD_STATIC Unary<Child> build() { return {}; }
};
template <typename I, typename P, typename O, typename Child, bool IS_FUSED = false>
struct BinaryOperation : detail::ParentCommon<BinaryType, Child, IS_FUSED>,
                         detail::BuildFromParams<detail::ParentCommon<BinaryType, Child, IS_FUSED>, P> {
    using InputType = I;
    using ParamsType = P;
    using OutputType = O;
    FK_HD_STATIC O exec(const I& input, const OperationData<Child, BinaryType>& opData) { return Child::exec(input, opData.params); }
};
template <typename I, typename P, typename BF, typename O, typename Child, bool IS_FUSED = false>
struct TernaryOperation : detail::ParentCommon<TernaryType, Child, IS_FUSED>,
                          detail::BuildFromParamsAndBack<detail::ParentCommon<TernaryType, Child, IS_FUSED>, P, BF> {
    using InputType = I;
    using ParamsType = P;
    using BackIOp = BF;
    using OutputType = O;
    FK_HD_STATIC O exec(const I& input, const OperationData<Child, TernaryType>& opData) {
        return Child::exec(input, opData.params, opData.backIOp);
    }
};
// A read or write with the thread-fusion tag enabled declares `template <uint ELEMS_PER_THREAD = 1> exec(...)`; the
// executors of this library always ask for one element (they vectorise by themselves where they know the layout).
template <typename RT, typename P, typename O, TF TFE, typename Child, bool IS_FUSED = false>
struct ReadOperation : detail::ParentCommon<ReadType, Child, IS_FUSED>, detail::BuildFromParams<detail::ParentCommon<ReadType, Child, IS_FUSED>, P> {
    using ReadDataType = RT;
    using ParamsType = P;
    using OutputType = O;
    static constexpr bool THREAD_FUSION = TFE == TF::ENABLED;
    template <uint ELEMS_PER_THREAD = 1>
    FK_HD_STATIC ThreadFusionType<RT, ELEMS_PER_THREAD, O> exec(const Point& thread, const OperationData<Child, ReadType>& opData) {
        if constexpr (THREAD_FUSION) {
            return Child::template exec<ELEMS_PER_THREAD>(thread, opData.params);
        } else {
            return Child::exec(thread, opData.params);
        }
    }
};
template <typename I, typename P, typename WT, TF TFE, typename Child, bool IS_FUSED = false>
struct WriteOperation : detail::ParentCommon<WriteType, Child, IS_FUSED>, detail::BuildFromParams<detail::ParentCommon<WriteType, Child, IS_FUSED>, P> {
    using InputType = I;
    using ParamsType = P;
    using WriteDataType = WT;
    static constexpr bool THREAD_FUSION = TFE == TF::ENABLED;
    template <uint ELEMS_PER_THREAD = 1>
    FK_HD_STATIC void exec(const Point& thread, const ThreadFusionType<I, ELEMS_PER_THREAD, I>& input, const OperationData<Child, WriteType>& opData) {
        if constexpr (THREAD_FUSION) {
            Child::template exec<ELEMS_PER_THREAD>(thread, input, opData.params);
        } else {
            Child::exec(thread, input, opData.params);
        }
    }
};
template <typename RT, typename P, typename B, typename O, typename Child, bool IS_FUSED = false>
struct ReadBackOperation : detail::ParentCommon<ReadBackType, Child, IS_FUSED>,
                           detail::BuildFromParamsAndBack<detail::ParentCommon<ReadBackType, Child, IS_FUSED>, P, B> {
    using ReadDataType = RT;
    using ParamsType = P;
    using BackIOp = B;
    using OutputType = O;
    static constexpr bool THREAD_FUSION = false;
    FK_HD_STATIC O exec(const Point& thread, const OperationData<Child, ReadBackType>& opData) {
        return Child::exec(thread, opData.params, opData.backIOp);
    }
};
} // namespace fk

// ---- the import macros: lists of the pieces below ---------------------------------------------------------------------
#define FK_PARENT_TYPE(NAME) using NAME = typename Parent::NAME;
#define FK_PARENT_FLAG(NAME) static constexpr bool NAME = Parent::NAME;
#define FK_PARENT_KIND FK_PARENT_TYPE(InstanceType) FK_PARENT_TYPE(InstantiableType) FK_PARENT_FLAG(IS_FUSED_OP)
#define FK_PARENT_BUILD_DATA                                                                                           \
    FK_PARENT_TYPE(OperationDataType)                                                                                  \
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return Parent::build(opData); }
#define FK_PARENT_BUILD_PARAMS FK_HD_STATIC InstantiableType build(const ParamsType& params) { return Parent::build(params); }
#define FK_PARENT_BUILD_PARAMS_BACK                                                                                    \
    FK_HD_STATIC InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return Parent::build(params, backIOp); }
#define FK_PARENT_EXEC_INPUT                                                                                           \
    FK_HD_STATIC OutputType exec(const InputType& input, const OperationDataType& opData) { return Parent::exec(input, opData); }

#define DECLARE_UNARY_PARENT                                                                                           \
    FK_PARENT_KIND FK_PARENT_TYPE(InputType) FK_PARENT_TYPE(OutputType)                                                \
    FK_HD_STATIC InstantiableType build() { return Parent::build(); }
#define DECLARE_BINARY_PARENT                                                                                          \
    FK_PARENT_KIND FK_PARENT_TYPE(InputType) FK_PARENT_TYPE(ParamsType) FK_PARENT_TYPE(OutputType)                     \
    FK_PARENT_BUILD_DATA FK_PARENT_BUILD_PARAMS FK_PARENT_EXEC_INPUT
#define DECLARE_TERNARY_PARENT                                                                                         \
    FK_PARENT_KIND FK_PARENT_TYPE(InputType) FK_PARENT_TYPE(ParamsType) FK_PARENT_TYPE(BackIOp) FK_PARENT_TYPE(OutputType) \
    FK_PARENT_BUILD_DATA FK_PARENT_BUILD_PARAMS_BACK FK_PARENT_EXEC_INPUT

#define DECLARE_READ_PARENT_BASIC                                                                                      \
    FK_PARENT_KIND FK_PARENT_TYPE(ReadDataType) FK_PARENT_TYPE(ParamsType) FK_PARENT_TYPE(OutputType)                  \
    FK_PARENT_FLAG(THREAD_FUSION) FK_PARENT_BUILD_DATA FK_PARENT_BUILD_PARAMS                                          \
    template <fk::uint ELEMS_PER_THREAD = 1>                                                                           \
    FK_HD_STATIC fk::ThreadFusionType<ReadDataType, ELEMS_PER_THREAD, OutputType> exec(const fk::Point& thread,        \
                                                                                       const OperationDataType& opData) { \
        return Parent::template exec<ELEMS_PER_THREAD>(thread, opData);                                                \
    }
// per-plane arrays of build() arguments -> an array of IOps (build_batch) or one BatchRead over them (build)
#define DECLARE_READ_PARENT_BATCH                                                                                      \
    template <size_t BATCH_N, typename FirstType, typename... ArrayTypes>                                              \
    static inline constexpr auto build_batch(const std::array<FirstType, BATCH_N>& first, const ArrayTypes&... arrays) { \
        return fk::BatchBuilders<typename Parent::Child>::build_batch(first, arrays...);                               \
    }                                                                                                                  \
    template <size_t BATCH_N, typename FirstType, typename... ArrayTypes>                                              \
    static inline constexpr auto build(const std::array<FirstType, BATCH_N>& first, const ArrayTypes&... arrays) {     \
        return fk::BatchBuilders<typename Parent::Child>::build(first, arrays...);                                     \
    }                                                                                                                  \
    template <size_t BATCH_N, typename DefaultValueType, typename FirstType, typename... ArrayTypes>                   \
    static inline constexpr auto build(const int& usedPlanes, const DefaultValueType& defaultValue,                    \
                                       const std::array<FirstType, BATCH_N>& first, const ArrayTypes&... arrays) {     \
        return fk::BatchBuilders<typename Parent::Child>::build(usedPlanes, defaultValue, first, arrays...);           \
    }
#define DECLARE_READ_PARENT DECLARE_READ_PARENT_BASIC DECLARE_READ_PARENT_BATCH

#define DECLARE_WRITE_PARENT_BASIC                                                                                     \
    FK_PARENT_KIND FK_PARENT_TYPE(InputType) FK_PARENT_TYPE(ParamsType) FK_PARENT_TYPE(WriteDataType)                  \
    FK_PARENT_FLAG(THREAD_FUSION) FK_PARENT_BUILD_DATA FK_PARENT_BUILD_PARAMS                                          \
    template <fk::uint ELEMS_PER_THREAD = 1>                                                                           \
    FK_HD_STATIC void exec(const fk::Point& thread, const fk::ThreadFusionType<InputType, ELEMS_PER_THREAD, InputType>& input, \
                           const OperationDataType& opData) {                                                          \
        Parent::template exec<ELEMS_PER_THREAD>(thread, input, opData);                                                \
    }
// per-plane arrays of build() arguments -> an array of IOps (build_batch) or one BatchWrite over them (build)
#define DECLARE_WRITE_PARENT_BATCH                                                                                     \
    template <size_t BATCH_N, typename FirstType, typename... ArrayTypes>                                              \
    static inline constexpr auto build_batch(const std::array<FirstType, BATCH_N>& first, const ArrayTypes&... arrays) { \
        return fk::BatchOperation::build_batch<typename Parent::Child>(first, arrays...);                              \
    }                                                                                                                  \
    template <size_t BATCH_N, typename FirstType, typename... ArrayTypes>                                              \
    static inline constexpr auto build(const std::array<FirstType, BATCH_N>& first, const ArrayTypes&... arrays) {     \
        return fk::BatchWrite<BATCH_N, typename Parent::Child>::build(first, arrays...);                               \
    }
#define DECLARE_WRITE_PARENT DECLARE_WRITE_PARENT_BASIC DECLARE_WRITE_PARENT_BATCH

#define DECLARE_READBACK_PARENT_ALIAS                                                                                  \
    FK_PARENT_KIND FK_PARENT_TYPE(ReadDataType) FK_PARENT_TYPE(ParamsType) FK_PARENT_TYPE(BackIOp) FK_PARENT_TYPE(OutputType) \
    FK_PARENT_FLAG(THREAD_FUSION) FK_PARENT_TYPE(OperationDataType)
#define DECLARE_READBACK_PARENT                                                                                        \
    DECLARE_READBACK_PARENT_ALIAS                                                                                      \
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return Parent::build(opData); }             \
    FK_PARENT_BUILD_PARAMS_BACK                                                                                        \
    FK_HD_STATIC OutputType exec(const fk::Point& thread, const OperationDataType& opData) { return Parent::exec(thread, opData); } \
    DECLARE_READ_PARENT_BATCH
#endif
