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
// A parent names the member types of one kind of operation (and the build()/exec(opData) forms that follow from them);
// the DECLARE_*_PARENT macro imports them into the operation.  Counterpart of the reference's
// core/execution_model/operation_model/parent_operations.h:23-281 and the batch halves of the read / write parents in
// batch_operations.h:408-450.  The operations of this library spell their members out directly, so these exist for
// operations written against the reference.
#ifndef FK_CORE_PARENT_OPERATIONS_H
#define FK_CORE_PARENT_OPERATIONS_H

#include "fk/core/operation_model.h"
#include "fk/core/thread_fusion_info.h"

namespace fk {
// OperationData<Child> is named with its kind spelled out: inside a parent the child is still incomplete, so its
// InstanceType cannot be asked for yet.
template <typename I, typename O, typename Child, bool IS_FUSED = false>
struct UnaryOperation {
    using InputType = I;
    using OutputType = O;
    using InstanceType = UnaryType;
    using InstantiableType = Unary<Child>;
    static constexpr bool IS_FUSED_OP = IS_FUSED;
    FK_HD_STATIC InstantiableType build() { return InstantiableType{}; }
};
#define DECLARE_UNARY_PARENT                                                                                           \
    using InputType = typename Parent::InputType;                                                                      \
    using OutputType = typename Parent::OutputType;                                                                    \
    using InstanceType = typename Parent::InstanceType;                                                                \
    using InstantiableType = typename Parent::InstantiableType;                                                        \
    static constexpr bool IS_FUSED_OP = Parent::IS_FUSED_OP;                                                           \
    FK_HD_STATIC InstantiableType build() { return Parent::build(); }

template <typename I, typename P, typename O, typename Child, bool IS_FUSED = false>
struct BinaryOperation {
    using InputType = I;
    using ParamsType = P;
    using OutputType = O;
    using InstanceType = BinaryType;
    using OperationDataType = OperationData<Child, BinaryType>;
    using InstantiableType = Binary<Child>;
    static constexpr bool IS_FUSED_OP = IS_FUSED;
    FK_HD_STATIC OutputType exec(const InputType& input, const OperationDataType& opData) { return Child::exec(input, opData.params); }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
};
#define DECLARE_BINARY_PARENT                                                                                          \
    using InputType = typename Parent::InputType;                                                                      \
    using ParamsType = typename Parent::ParamsType;                                                                    \
    using OutputType = typename Parent::OutputType;                                                                    \
    using InstanceType = typename Parent::InstanceType;                                                                \
    using OperationDataType = typename Parent::OperationDataType;                                                      \
    using InstantiableType = typename Parent::InstantiableType;                                                        \
    static constexpr bool IS_FUSED_OP = Parent::IS_FUSED_OP;                                                           \
    FK_HD_STATIC OutputType exec(const InputType& input, const OperationDataType& opData) { return Parent::exec(input, opData); } \
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return Parent::build(opData); }             \
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return Parent::build(params); }

template <typename I, typename P, typename BF, typename O, typename Child, bool IS_FUSED = false>
struct TernaryOperation {
    using InputType = I;
    using ParamsType = P;
    using BackIOp = BF;
    using OutputType = O;
    using InstanceType = TernaryType;
    using OperationDataType = OperationData<Child, TernaryType>;
    using InstantiableType = Ternary<Child>;
    static constexpr bool IS_FUSED_OP = IS_FUSED;
    FK_HD_STATIC OutputType exec(const InputType& input, const OperationDataType& opData) { return Child::exec(input, opData.params, opData.backIOp); }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return InstantiableType{ { params, backIOp } }; }
};
#define DECLARE_TERNARY_PARENT                                                                                         \
    using InputType = typename Parent::InputType;                                                                      \
    using ParamsType = typename Parent::ParamsType;                                                                    \
    using BackIOp = typename Parent::BackIOp;                                                                          \
    using OutputType = typename Parent::OutputType;                                                                    \
    using InstanceType = typename Parent::InstanceType;                                                                \
    using OperationDataType = typename Parent::OperationDataType;                                                      \
    using InstantiableType = typename Parent::InstantiableType;                                                        \
    static constexpr bool IS_FUSED_OP = Parent::IS_FUSED_OP;                                                           \
    FK_HD_STATIC OutputType exec(const InputType& input, const OperationDataType& opData) { return Parent::exec(input, opData); } \
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return Parent::build(opData); }             \
    FK_HD_STATIC InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return Parent::build(params, backIOp); }

// A read with the thread-fusion tag enabled declares `template <uint ELEMS_PER_THREAD = 1> exec(thread, params)`; the
// executors of this library always ask for one element (they vectorise by themselves where they know the layout).
template <typename RT, typename P, typename O, TF TFE, typename Child_, bool IS_FUSED = false>
struct ReadOperation {
    using Child = Child_;
    using ReadDataType = RT;
    using ParamsType = P;
    using OutputType = O;
    using InstanceType = ReadType;
    using OperationDataType = OperationData<Child_, ReadType>;
    using InstantiableType = Read<Child_>;
    static constexpr bool IS_FUSED_OP = IS_FUSED;
    static constexpr bool THREAD_FUSION = static_cast<bool>(TFE);
    template <uint ELEMS_PER_THREAD = 1>
    FK_HD_STATIC ThreadFusionType<ReadDataType, ELEMS_PER_THREAD, OutputType> exec(const Point& thread, const OperationDataType& opData) {
        if constexpr (THREAD_FUSION) {
            return Child_::template exec<ELEMS_PER_THREAD>(thread, opData.params);
        } else {
            return Child_::exec(thread, opData.params);
        }
    }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
};
#define DECLARE_READ_PARENT_BASIC                                                                                      \
    using ReadDataType = typename Parent::ReadDataType;                                                                \
    using ParamsType = typename Parent::ParamsType;                                                                    \
    using OutputType = typename Parent::OutputType;                                                                    \
    using InstanceType = typename Parent::InstanceType;                                                                \
    using OperationDataType = typename Parent::OperationDataType;                                                      \
    using InstantiableType = typename Parent::InstantiableType;                                                        \
    static constexpr bool IS_FUSED_OP = Parent::IS_FUSED_OP;                                                           \
    static constexpr bool THREAD_FUSION = Parent::THREAD_FUSION;                                                       \
    template <fk::uint ELEMS_PER_THREAD = 1>                                                                           \
    FK_HD_STATIC fk::ThreadFusionType<ReadDataType, ELEMS_PER_THREAD, OutputType> exec(const fk::Point& thread,        \
                                                                                       const OperationDataType& opData) { \
        return Parent::template exec<ELEMS_PER_THREAD>(thread, opData);                                                \
    }                                                                                                                  \
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return Parent::build(opData); }             \
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return Parent::build(params); }
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
#define DECLARE_READ_PARENT                                                                                            \
    DECLARE_READ_PARENT_BASIC                                                                                          \
    DECLARE_READ_PARENT_BATCH

template <typename I, typename P, typename WT, TF TFE, typename Child_, bool IS_FUSED = false>
struct WriteOperation {
    using Child = Child_;
    using InputType = I;
    using ParamsType = P;
    using WriteDataType = WT;
    using InstanceType = WriteType;
    using OperationDataType = OperationData<Child_, WriteType>;
    using InstantiableType = Write<Child_>;
    static constexpr bool IS_FUSED_OP = IS_FUSED;
    static constexpr bool THREAD_FUSION = static_cast<bool>(TFE);
    template <uint ELEMS_PER_THREAD = 1>
    FK_HD_STATIC void exec(const Point& thread, const ThreadFusionType<InputType, ELEMS_PER_THREAD, InputType>& input, const OperationDataType& opData) {
        if constexpr (THREAD_FUSION) {
            Child_::template exec<ELEMS_PER_THREAD>(thread, input, opData.params);
        } else {
            Child_::exec(thread, input, opData.params);
        }
    }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
};
#define DECLARE_WRITE_PARENT_BASIC                                                                                     \
    using InputType = typename Parent::InputType;                                                                      \
    using ParamsType = typename Parent::ParamsType;                                                                    \
    using WriteDataType = typename Parent::WriteDataType;                                                              \
    using InstanceType = typename Parent::InstanceType;                                                                \
    using OperationDataType = typename Parent::OperationDataType;                                                      \
    using InstantiableType = typename Parent::InstantiableType;                                                        \
    static constexpr bool IS_FUSED_OP = Parent::IS_FUSED_OP;                                                           \
    static constexpr bool THREAD_FUSION = Parent::THREAD_FUSION;                                                       \
    template <fk::uint ELEMS_PER_THREAD = 1>                                                                           \
    FK_HD_STATIC void exec(const fk::Point& thread, const fk::ThreadFusionType<InputType, ELEMS_PER_THREAD, InputType>& input, \
                           const OperationDataType& opData) {                                                          \
        Parent::template exec<ELEMS_PER_THREAD>(thread, input, opData);                                                \
    }                                                                                                                  \
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return Parent::build(opData); }             \
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return Parent::build(params); }
#define DECLARE_WRITE_PARENT_BATCH                                                                                     \
    template <size_t BATCH_N, typename FirstType, typename... ArrayTypes>                                              \
    static inline constexpr auto build_batch(const std::array<FirstType, BATCH_N>& first, const ArrayTypes&... arrays) { \
        return fk::BatchOperation::build_batch<typename Parent::Child>(first, arrays...);                              \
    }                                                                                                                  \
    template <size_t BATCH_N, typename FirstType, typename... ArrayTypes>                                              \
    static inline constexpr auto build(const std::array<FirstType, BATCH_N>& first, const ArrayTypes&... arrays) {     \
        return fk::BatchWrite<BATCH_N, typename Parent::Child>::build(first, arrays...);                               \
    }
#define DECLARE_WRITE_PARENT                                                                                           \
    DECLARE_WRITE_PARENT_BASIC                                                                                         \
    DECLARE_WRITE_PARENT_BATCH

template <typename RT, typename P, typename B, typename O, typename Child_, bool IS_FUSED = false>
struct ReadBackOperation {
    using Child = Child_;
    using ReadDataType = RT;
    using ParamsType = P;
    using BackIOp = B;
    using OutputType = O;
    using InstanceType = ReadBackType;
    using OperationDataType = OperationData<Child_, ReadBackType>;
    using InstantiableType = ReadBack<Child_>;
    static constexpr bool IS_FUSED_OP = IS_FUSED;
    static constexpr bool THREAD_FUSION = false;
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return Child_::exec(thread, opData.params, opData.backIOp); }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return InstantiableType{ { params, backIOp } }; }
};
#define DECLARE_READBACK_PARENT_ALIAS                                                                                  \
    using ReadDataType = typename Parent::ReadDataType;                                                                \
    using ParamsType = typename Parent::ParamsType;                                                                    \
    using BackIOp = typename Parent::BackIOp;                                                                          \
    using OutputType = typename Parent::OutputType;                                                                    \
    using InstanceType = typename Parent::InstanceType;                                                                \
    using OperationDataType = typename Parent::OperationDataType;                                                      \
    using InstantiableType = typename Parent::InstantiableType;                                                        \
    static constexpr bool IS_FUSED_OP = Parent::IS_FUSED_OP;                                                           \
    static constexpr bool THREAD_FUSION = Parent::THREAD_FUSION;
#define DECLARE_READBACK_PARENT                                                                                        \
    DECLARE_READBACK_PARENT_ALIAS                                                                                      \
    FK_HD_STATIC OutputType exec(const fk::Point& thread, const OperationDataType& opData) { return Parent::exec(thread, opData); } \
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return Parent::build(opData); }             \
    FK_HD_STATIC InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return Parent::build(params, backIOp); } \
    DECLARE_READ_PARENT_BATCH
} // namespace fk
#endif
