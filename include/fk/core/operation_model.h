// The operation model: operation kinds, instantiable operations (IOps) with .then(), OperationTuple,
// FusedOperation, the Fuser and batch (per-plane) reads.
//
// API counterpart of the reference's core/execution_model/operation_model/*:
//   kinds and traits          operation_types.h:23-186
//   OperationData             operation_data.h:79-159   (members `params` and, for ReadBack/Ternary, `backIOp`)
//   IOp wrappers, then()      instantiable_operations.h:44-212
//   OperationTuple            operation_tuple.h:22-205  (members `instance`, `next`; Unary operations store nothing)
//   FusedOperation            fused_operation.h:136-326 (a chain behaves as one Read, Unary or Binary operation)
//   Fuser                     iop_fuser.h:22-143        (batch x non-batch combinations)
//   BatchRead                 batch_operations.h:87-260 (`opData[BATCH]`, PlanePolicy, activeThreads = max w, max h, BATCH)
// An operation is a struct of static functions; an IOp is a trivially copyable value that carries its runtime
// parameters, so a whole chain can be handed to a kernel by value.
#ifndef FK_CORE_OPERATION_MODEL_H
#define FK_CORE_OPERATION_MODEL_H

#include <array>

#include "fk/core/data.h"
#include "fk/core/type_utils.h"

namespace fk {

// ---- kinds --------------------------------------------------------------------------------------------------
struct ReadType {};
struct ReadBackType {};
struct UnaryType {};
struct BinaryType {};
struct TernaryType {};
struct MidWriteType {};
struct WriteType {};

enum class TF : bool { ENABLED = true, DISABLED = false };

namespace detail {
template <typename T, typename = void>
struct KindOf {
    using type = void;
};
template <typename T>
struct KindOf<T, std::void_t<typename T::InstanceType>> {
    using type = typename T::InstanceType;
};
template <typename T, typename Kind>
constexpr bool is_kind = std::is_same_v<typename KindOf<T>::type, Kind>;
} // namespace detail

template <typename T> constexpr bool isOperation = !std::is_void_v<typename detail::KindOf<T>::type>;
template <typename T> constexpr bool isReadType = detail::is_kind<T, ReadType>;
template <typename T> constexpr bool isReadBackType = detail::is_kind<T, ReadBackType>;
template <typename T> constexpr bool isAnyReadType = isReadType<T> || isReadBackType<T>;
template <typename T> constexpr bool isUnaryType = detail::is_kind<T, UnaryType>;
template <typename T> constexpr bool isBinaryType = detail::is_kind<T, BinaryType>;
template <typename T> constexpr bool isTernaryType = detail::is_kind<T, TernaryType>;
template <typename T> constexpr bool isWriteType = detail::is_kind<T, WriteType>;
template <typename T> constexpr bool isMidWriteType = detail::is_kind<T, MidWriteType>;
template <typename T> constexpr bool isAnyWriteType = isWriteType<T> || isMidWriteType<T>;
// the same as class templates, for use in template argument lists
template <typename T> struct IsReadType : std::bool_constant<isReadType<T>> {};
template <typename T> struct IsReadBackType : std::bool_constant<isReadBackType<T>> {};
template <typename T> struct IsUnaryType : std::bool_constant<isUnaryType<T>> {};
template <typename T> struct IsBinaryType : std::bool_constant<isBinaryType<T>> {};
template <typename T> struct IsTernaryType : std::bool_constant<isTernaryType<T>> {};
template <typename T> struct IsMidWriteType : std::bool_constant<isMidWriteType<T>> {};
template <typename T> struct IsWriteType : std::bool_constant<isWriteType<T>> {};
using WriteTypeList = TypeList<WriteType, MidWriteType>;
template <typename T> constexpr bool isComputeType = isUnaryType<T> || isBinaryType<T> || isTernaryType<T>;
template <typename... Ts> constexpr bool allUnaryTypes = (isUnaryType<Ts> && ...);
template <typename... Ts> constexpr bool notAllUnaryTypes = !allUnaryTypes<Ts...>;
template <typename... Ts> constexpr bool noneWriteType = (!isWriteType<Ts> && ...);
template <typename... Ts> constexpr bool noneMidWriteType = (!isMidWriteType<Ts> && ...);
template <typename... Ts> constexpr bool noneAnyWriteType = (!isAnyWriteType<Ts> && ...);

// A restriction for filtered_index_sequence_t over a list of kind tags: the kinds that carry parameters.
struct NotUnaryRestriction {
    template <typename Kind>
    static constexpr bool complies() {
        return !std::is_same_v<Kind, UnaryType>;
    }
};

template <typename IOp> using GetInputType_t = typename IOp::Operation::InputType;
template <typename IOp> using GetOutputType_t = typename IOp::Operation::OutputType;

namespace detail {
template <typename T, typename = void>
struct IsBuilderOnly : std::false_type {};
template <typename T>
struct IsBuilderOnly<T, std::enable_if_t<T::BUILDER_ONLY>> : std::true_type {};
template <typename T, typename = void>
struct HasBatch : std::false_type {};
template <typename T>
struct HasBatch<T, std::void_t<decltype(T::BATCH)>> : std::true_type {};
template <typename T, typename = void>
struct IsFused : std::false_type {};
template <typename T>
struct IsFused<T, std::enable_if_t<T::IS_FUSED_OP>> : std::true_type {};
} // namespace detail
// An operation is complete when it can execute; Crop<void>, Resize<..., void> are builders waiting for their back read.
template <typename T> constexpr bool isCompleteOperation = isOperation<T> && !detail::IsBuilderOnly<T>::value;
template <typename Op> constexpr bool isBatchOperation = detail::HasBatch<Op>::value;
template <typename Op> using is_fused_operation = detail::IsFused<Op>;

// ---- OperationData ------------------------------------------------------------------------------------------
template <typename Op, typename Kind = typename Op::InstanceType>
struct OperationData {
    typename Op::ParamsType params;
};
template <typename Op>
struct OperationData<Op, UnaryType> {};
template <typename Op>
struct OperationData<Op, ReadBackType> {
    typename Op::ParamsType params;
    typename Op::BackIOp backIOp;
};
template <typename Op>
struct OperationData<Op, TernaryType> {
    typename Op::ParamsType params;
    typename Op::BackIOp backIOp;
};

// ---- instantiable operations ------------------------------------------------------------------------------------
struct Fuser;

#define FK_IOP_COMMON(KIND)                                                                                            \
    using Operation = Operation_t;                                                                                     \
    using InstanceType = KIND;                                                                                         \
    template <typename IT>                                                                                             \
    static constexpr bool is = std::is_same_v<IT, KIND>;
#define FK_IOP_THEN                                                                                                    \
    template <typename ContinuationIOp, typename Fuser_t = Fuser>                                                      \
    inline constexpr auto then(const ContinuationIOp& cIOp) const {                                                    \
        return Fuser_t::fuse(*this, cIOp);                                                                             \
    }                                                                                                                  \
    template <typename ContinuationIOp, typename... ContinuationIOps>                                                  \
    inline constexpr auto then(const ContinuationIOp& cIOp, const ContinuationIOps&... cIOps) const {                  \
        return then(cIOp).then(cIOps...);                                                                              \
    }

template <typename Operation_t>
struct ReadInstantiableOperation final : public OperationData<Operation_t> {
    FK_IOP_COMMON(ReadType)
    FK_IOP_THEN
    FK_HD_CNST ActiveThreads getActiveThreads() const { return Operation::getActiveThreads(*this); }
};
template <typename Operation_t>
struct ReadBackInstantiableOperation final : public OperationData<Operation_t> {
    FK_IOP_COMMON(ReadBackType)
    FK_IOP_THEN
    FK_HD_CNST ActiveThreads getActiveThreads() const { return Operation::getActiveThreads(*this); }
};
template <typename Operation_t>
struct UnaryInstantiableOperation {
    FK_IOP_COMMON(UnaryType)
    FK_IOP_THEN
};
template <typename Operation_t>
struct BinaryInstantiableOperation final : public OperationData<Operation_t> {
    FK_IOP_COMMON(BinaryType)
    FK_IOP_THEN
};
template <typename Operation_t>
struct TernaryInstantiableOperation final : public OperationData<Operation_t> {
    FK_IOP_COMMON(TernaryType)
    FK_IOP_THEN
};
template <typename Operation_t>
struct MidWriteInstantiableOperation final : public OperationData<Operation_t> {
    FK_IOP_COMMON(MidWriteType)
    FK_IOP_THEN
};
template <typename Operation_t>
struct WriteInstantiableOperation final : public OperationData<Operation_t> {
    FK_IOP_COMMON(WriteType)
};
#undef FK_IOP_COMMON
#undef FK_IOP_THEN

template <typename Op> using Read = ReadInstantiableOperation<Op>;
template <typename Op> using ReadBack = ReadBackInstantiableOperation<Op>;
template <typename Op> using Unary = UnaryInstantiableOperation<Op>;
template <typename Op> using Binary = BinaryInstantiableOperation<Op>;
template <typename Op> using Ternary = TernaryInstantiableOperation<Op>;
template <typename Op> using MidWrite = MidWriteInstantiableOperation<Op>;
template <typename Op> using Write = WriteInstantiableOperation<Op>;

namespace detail {
template <typename Op, typename Kind>
struct InstantiableFor;
template <typename Op> struct InstantiableFor<Op, ReadType> { using type = Read<Op>; };
template <typename Op> struct InstantiableFor<Op, ReadBackType> { using type = ReadBack<Op>; };
template <typename Op> struct InstantiableFor<Op, UnaryType> { using type = Unary<Op>; };
template <typename Op> struct InstantiableFor<Op, BinaryType> { using type = Binary<Op>; };
template <typename Op> struct InstantiableFor<Op, TernaryType> { using type = Ternary<Op>; };
template <typename Op> struct InstantiableFor<Op, MidWriteType> { using type = MidWrite<Op>; };
template <typename Op> struct InstantiableFor<Op, WriteType> { using type = Write<Op>; };
} // namespace detail
template <typename Op>
using Instantiable = typename detail::InstantiableFor<Op, typename Op::InstanceType>::type;

// IOp of `Op` from its OperationData (a no-op conversion: the IOp only adds static members).
template <typename Op>
FK_HD_CNST Instantiable<Op> toIOp(const OperationData<Op>& data) {
    if constexpr (isUnaryType<Op>) {
        return Instantiable<Op>{};
    } else {
        return Instantiable<Op>{ data };
    }
}

// Run one compute IOp on a value held in registers (operation_types.h:126-136).
template <typename IOp>
FK_HD_CNST GetOutputType_t<IOp> compute(const GetInputType_t<IOp>& input, const IOp& iOp) {
    static_assert(isComputeType<IOp>, "compute() takes Unary, Binary or Ternary operations");
    if constexpr (isUnaryType<IOp>) {
        return IOp::Operation::exec(input);
    } else {
        return IOp::Operation::exec(input, iOp);
    }
}

// ---- OperationTuple -----------------------------------------------------------------------------------------
template <typename... Operations>
struct OperationTuple;

namespace detail {
template <typename Op, bool STORED = !isUnaryType<Op>>
struct TupleInstance {
    OperationData<Op> instance;
};
template <typename Op>
struct TupleInstance<Op, false> {};
template <bool STORED, typename... Rest>
struct TupleNext {
    OperationTuple<Rest...> next;
};
template <typename... Rest>
struct TupleNext<false, Rest...> {};
} // namespace detail

template <typename Operation_t, typename... Rest>
struct OperationTuple<Operation_t, Rest...>
    : detail::TupleInstance<Operation_t>, detail::TupleNext<(sizeof...(Rest) > 0) && !allUnaryTypes<Rest...>, Rest...> {
    using Operation = Operation_t;
    static constexpr bool HAS_INSTANCE = !isUnaryType<Operation_t>;
    static constexpr bool HAS_NEXT = (sizeof...(Rest) > 0) && !allUnaryTypes<Rest...>;
    static constexpr bool HAS_REST = sizeof...(Rest) > 0;
    using Next = OperationTuple<Rest...>; // the type list of the tail (a member `next` exists only where it holds data)
    enum { size = sizeof...(Rest) + 1 };
};

namespace detail {
template <typename List>
struct Rest;
template <typename First, typename... Others>
struct Rest<OperationTuple<First, Others...>> {
    using type = OperationTuple<Others...>;
};
template <typename A, typename B>
struct TupleCat;
template <typename... As, typename... Bs>
struct TupleCat<OperationTuple<As...>, OperationTuple<Bs...>> {
    using type = OperationTuple<As..., Bs...>;
};

// The tail of a tuple as a value; tails made only of Unary operations hold no data.
template <typename Op, typename... Rest_>
FK_HD_CNST OperationTuple<Rest_...> tuple_tail(const OperationTuple<Op, Rest_...>& t) {
    if constexpr (OperationTuple<Op, Rest_...>::HAS_NEXT) {
        return t.next;
    } else {
        return OperationTuple<Rest_...>{};
    }
}

// Copies the stored instances of `a` followed by those of `b` into `out` (their concatenation).
template <typename Out, typename A, typename B>
FK_HD_CNST void tuple_fill(Out& out, const A& a, const B& b) {
    if constexpr (A::HAS_INSTANCE) out.instance = a.instance;
    if constexpr (Out::HAS_NEXT) {
        if constexpr (A::HAS_REST) {
            tuple_fill(out.next, tuple_tail(a), b);
        } else {
            out.next = b;
        }
    }
}
} // namespace detail

template <typename... As, typename... Bs>
FK_HD_CNST OperationTuple<As..., Bs...> operation_tuple_cat(const OperationTuple<As...>& a, const OperationTuple<Bs...>& b) {
    OperationTuple<As..., Bs...> out{};
    detail::tuple_fill(out, a, b);
    return out;
}

template <typename... As, typename... Bs>
FK_HD_CNST OperationTuple<As..., Bs...> cat(const OperationTuple<As...>& a, const OperationTuple<Bs...>& b) {
    return operation_tuple_cat(a, b);
}

namespace detail {
template <typename Tuple_>
FK_HD_CNST void tuple_assign(Tuple_&) {}
template <typename Tuple_, typename First, typename... More>
FK_HD_CNST void tuple_assign(Tuple_& t, const First& first, const More&... more) {
    if constexpr (Tuple_::HAS_INSTANCE) {
        t.instance = first;
        if constexpr (sizeof...(More) > 0) tuple_assign(t.next, more...);
    } else {
        tuple_assign(t.next, first, more...);
    }
}
} // namespace detail
// An OperationTuple of the given operations, from the OperationData of those that have any (in order).
template <typename... Operations, typename... Datas>
FK_HD_CNST OperationTuple<Operations...> make_operation_tuple_(const Datas&... datas) {
    static_assert(((isUnaryType<Operations> ? 0 : 1) + ...) == sizeof...(Datas), "One OperationData per operation that is not Unary.");
    OperationTuple<Operations...> t{};
    detail::tuple_assign(t, datas...);
    return t;
}

// OperationData of element INDEX of the tuple; Unary elements have none.
template <int INDEX, typename... Ops>
FK_HD_CNST auto get(const OperationTuple<Ops...>& t) {
    static_assert(INDEX >= 0 && INDEX < static_cast<int>(sizeof...(Ops)), "Index out of range.");
    if constexpr (INDEX == 0) {
        static_assert(OperationTuple<Ops...>::HAS_INSTANCE, "This is an Unary operation, and it does not have params.");
        return t.instance;
    } else {
        return get<INDEX - 1>(t.next);
    }
}

namespace detail {
template <int INDEX, typename First, typename... Rest_>
struct TupleElement<INDEX, OperationTuple<First, Rest_...>> {
    using type = typename TupleElement<INDEX - 1, OperationTuple<Rest_...>>::type;
};
template <typename First, typename... Rest_>
struct TupleElement<0, OperationTuple<First, Rest_...>> {
    using type = First;
};
template <size_t N, typename... Ops>
struct TypeAtImpl<N, OperationTuple<Ops...>> : TypeAtImpl<N, TypeList<Ops...>> {};
template <int INDEX, typename TupleLike>
struct ElementOf : TupleElement<INDEX, TupleLike> {};
template <int INDEX, typename... Types>
struct ElementOf<INDEX, TypeList<Types...>> : TypeAtImpl<static_cast<size_t>(INDEX), TypeList<Types...>> {};
} // namespace detail
template <int INDEX, typename TupleLike>
using get_type_t = typename detail::ElementOf<INDEX, TupleLike>::type;

// ---- FusedOperation -----------------------------------------------------------------------------------------
namespace detail {
// One operation of a fused chain applied to `input`: compute operations transform it; a write in the middle of a chain
// stores it at `thread` and hands it on unchanged (a fused write-then-compute operation hands on its own result).
template <typename Op, typename Input, typename Instance>
FK_HD_CNST auto chain_step(const Point& thread, const Input& input, const Instance& holder) {
    if constexpr (isUnaryType<Op>) {
        return Op::exec(input);
    } else if constexpr (isWriteType<Op>) {
        Op::exec(thread, input, holder.instance);
        return input;
    } else if constexpr (isMidWriteType<Op>) {
        return Op::exec(thread, input, holder.instance);
    } else {
        static_assert(isComputeType<Op>, "Only compute and write operations can follow the first operation of a fused chain.");
        return Op::exec(input, holder.instance);
    }
}
// Runs the operations of a tuple in order on `input`.  The tuple is only ever walked by reference, so a long chain
// stays in the registers (or kernel-argument scalars) it arrived in.
template <typename Input, typename Op, typename... Rest_>
FK_HD_CNST auto tuple_compute(const Point& thread, const Input& input, const OperationTuple<Op, Rest_...>& t) {
    using Tuple = OperationTuple<Op, Rest_...>;
    if constexpr (sizeof...(Rest_) == 0) {
        return chain_step<Op>(thread, input, t);
    } else if constexpr (Tuple::HAS_NEXT) {
        return tuple_compute(thread, chain_step<Op>(thread, input, t), t.next);
    } else { // the rest is Unary only and holds no data
        return tuple_compute(thread, chain_step<Op>(thread, input, t), OperationTuple<Rest_...>{});
    }
}
template <typename Input, typename Op, typename... Rest_>
FK_HD_CNST auto tuple_compute(const Input& input, const OperationTuple<Op, Rest_...>& t) {
    static_assert(noneAnyWriteType<Op, Rest_...>, "A chain with writes needs the thread it runs for.");
    return tuple_compute(Point(), input, t);
}
// Same, starting after the first element of the tuple (the read of a fused read chain).
template <typename Input, typename Op, typename... Rest_>
FK_HD_CNST auto tuple_compute_after_first(const Point& thread, const Input& input, const OperationTuple<Op, Rest_...>& t) {
    if constexpr (OperationTuple<Op, Rest_...>::HAS_NEXT) {
        return tuple_compute(thread, input, t.next);
    } else {
        return tuple_compute(thread, input, OperationTuple<Rest_...>{});
    }
}
template <typename... Ops>
struct LastOf;
template <typename Op>
struct LastOf<Op> {
    using type = Op;
};
template <typename Op, typename... Rest_>
struct LastOf<Op, Rest_...> {
    using type = typename LastOf<Rest_...>::type;
};
template <typename Op, typename... Rest_>
struct FirstOf {
    using type = Op;
};
// what a chain hands on after its last operation: that operation's output, or for a write the value it stored
template <typename Op, typename = void>
struct HandsOn {
    using type = typename Op::OutputType;
};
template <typename Op>
struct HandsOn<Op, std::enable_if_t<isWriteType<Op>>> {
    using type = typename Op::InputType;
};
template <typename... Ops>
using ChainOutput_t = typename HandsOn<typename LastOf<Ops...>::type>::type;
} // namespace detail

template <typename Enabler, typename... Operations>
struct FusedOperation_;

template <typename... Operations>
using FusedOperation = FusedOperation_<void, Operations...>;

// A chain that starts with a read: behaves as one Read operation.
template <typename FirstOp, typename... ComputeOps>
struct FusedOperation_<std::enable_if_t<isAnyReadType<FirstOp>>, FirstOp, ComputeOps...> {
private:
    using SelfType = FusedOperation_<void, FirstOp, ComputeOps...>;

public:
    FK_STATIC_STRUCT(FusedOperation_, SelfType)
    using Operations = OperationTuple<FirstOp, ComputeOps...>;
    using ParamsType = OperationTuple<FirstOp, ComputeOps...>;
    using ReadDataType = typename FirstOp::ReadDataType;
    using OutputType = detail::ChainOutput_t<FirstOp, ComputeOps...>;
    using InstanceType = ReadType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Read<SelfType>;
    static constexpr bool IS_FUSED_OP = true;
    static constexpr bool THREAD_FUSION = false;
    using HeadOperation = FirstOp;

    FK_HD_STATIC OutputType exec(const Point& thread, const ParamsType& params) {
        if constexpr (sizeof...(ComputeOps) == 0) {
            return FirstOp::exec(thread, params.instance);
        } else {
            return detail::tuple_compute_after_first(thread, FirstOp::exec(thread, params.instance), params);
        }
    }
    FK_HD_STATIC OutputType exec(const Point& thread, const OperationDataType& opData) { return exec(thread, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point& thread, const OperationDataType& opData) { return FirstOp::num_elems_x(thread, opData.params.instance); }
    FK_HD_STATIC uint num_elems_y(const Point& thread, const OperationDataType& opData) { return FirstOp::num_elems_y(thread, opData.params.instance); }
    FK_HD_STATIC uint num_elems_z(const Point& thread, const OperationDataType& opData) { return FirstOp::num_elems_z(thread, opData.params.instance); }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) { return FirstOp::getActiveThreads(opData.params.instance); }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
    template <size_t BATCH_N>
    static inline constexpr auto build(const std::array<InstantiableType, BATCH_N>& iOps);
};

// A chain of Unary operations only: behaves as one Unary operation.
template <typename FirstOp, typename... Ops>
struct FusedOperation_<std::enable_if_t<allUnaryTypes<FirstOp, Ops...>>, FirstOp, Ops...> {
private:
    using SelfType = FusedOperation_<void, FirstOp, Ops...>;

public:
    FK_STATIC_STRUCT(FusedOperation_, SelfType)
    using Operations = OperationTuple<FirstOp, Ops...>;
    using InputType = typename FirstOp::InputType;
    using OutputType = typename detail::LastOf<FirstOp, Ops...>::type::OutputType;
    using InstanceType = UnaryType;
    using InstantiableType = Unary<SelfType>;
    static constexpr bool IS_FUSED_OP = true;
    FK_HD_STATIC OutputType exec(const InputType& input) { return detail::tuple_compute(input, Operations{}); }
    FK_HD_STATIC InstantiableType build() { return InstantiableType{}; }
};

// A chain of compute operations with parameters: behaves as one Binary operation.
template <typename FirstOp, typename... Ops>
struct FusedOperation_<std::enable_if_t<isComputeType<FirstOp> && !allUnaryTypes<FirstOp, Ops...>>, FirstOp, Ops...> {
private:
    using SelfType = FusedOperation_<void, FirstOp, Ops...>;

public:
    FK_STATIC_STRUCT(FusedOperation_, SelfType)
    using Operations = OperationTuple<FirstOp, Ops...>;
    using ParamsType = OperationTuple<FirstOp, Ops...>;
    using InputType = typename FirstOp::InputType;
    using OutputType = typename detail::LastOf<FirstOp, Ops...>::type::OutputType;
    using InstanceType = BinaryType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Binary<SelfType>;
    static constexpr bool IS_FUSED_OP = true;
    FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) { return detail::tuple_compute(input, params); }
    FK_HD_STATIC OutputType exec(const InputType& input, const OperationDataType& opData) { return exec(input, opData.params); }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
};

// A chain that starts with a write: stores its input at the thread's position, runs the rest on it and hands the result
// on, so as a whole it behaves as one MidWrite operation.
template <typename FirstOp, typename... Ops>
struct FusedOperation_<std::enable_if_t<isAnyWriteType<FirstOp>>, FirstOp, Ops...> {
private:
    using SelfType = FusedOperation_<void, FirstOp, Ops...>;

public:
    FK_STATIC_STRUCT(FusedOperation_, SelfType)
    using ParamsType = OperationTuple<FirstOp, Ops...>;
    using InputType = typename FirstOp::InputType;
    using OutputType = detail::ChainOutput_t<FirstOp, Ops...>;
    using WriteDataType = typename FirstOp::WriteDataType;
    using InstanceType = MidWriteType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = MidWrite<SelfType>;
    static constexpr bool IS_FUSED_OP = true;
    static constexpr bool THREAD_FUSION = false;
    FK_HD_STATIC OutputType exec(const Point& thread, const InputType& input, const ParamsType& params) {
        return detail::tuple_compute(thread, input, params);
    }
    FK_HD_STATIC OutputType exec(const Point& thread, const InputType& input, const OperationDataType& opData) {
        return exec(thread, input, opData.params);
    }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
};

namespace detail {
// One IOp as an OperationTuple: fused IOps contribute their whole tuple, so chains never nest.
template <typename IOp>
FK_HD_CNST auto iop_to_tuple(const IOp& iOp) {
    using Op = typename IOp::Operation;
    if constexpr (IsFused<Op>::value) {
        if constexpr (isUnaryType<IOp>) {
            return typename Op::Operations{};
        } else {
            return iOp.params;
        }
    } else {
        OperationTuple<Op> t{};
        if constexpr (!isUnaryType<IOp>) {
            t.instance = static_cast<const OperationData<Op>&>(iOp);
        }
        return t;
    }
}
template <typename... Ops>
FK_HD_CNST auto tuple_to_iop(const OperationTuple<Ops...>& t) {
    using Fused = FusedOperation<Ops...>;
    if constexpr (isUnaryType<Fused>) {
        return Unary<Fused>{};
    } else {
        return Fused::build(t);
    }
}
} // namespace detail

// The OperationTuple of a sequence of IOps; fused IOps contribute their elements.
template <typename IOp>
FK_HD_CNST auto iOpsToOperationTuple(const IOp& iOp) {
    return detail::iop_to_tuple(iOp);
}
template <typename IOp, typename... IOps>
FK_HD_CNST auto iOpsToOperationTuple(const IOp& iOp, const IOps&... iOps) {
    return operation_tuple_cat(detail::iop_to_tuple(iOp), iOpsToOperationTuple(iOps...));
}

// An all-Unary FusedOperation carries its operations as a type only; any other one as a tuple of their data.
template <typename Operation, typename = void>
struct IsAllUnaryFusedOperation : std::false_type {};
template <typename Operation>
struct IsAllUnaryFusedOperation<Operation, std::enable_if_t<detail::IsFused<Operation>::value && isUnaryType<Operation>>> : std::true_type {};
template <typename Operation>
constexpr bool isAllUnaryFusedOperation = IsAllUnaryFusedOperation<Operation>::value;
template <typename Operation>
constexpr bool isNotAllUnaryFusedOperation = !isAllUnaryFusedOperation<Operation>;

// Both directions between a fused IOp and the OperationTuple it stands for.
template <typename FusedIOp>
struct InstantiableFusedOperationToOperationTuple {
    static_assert(detail::IsFused<typename FusedIOp::Operation>::value, "Not a fused operation.");
    FK_HD_STATIC auto value(const FusedIOp& iOp) { return detail::iop_to_tuple(iOp); }
};
template <typename Tuple_>
struct OperationTupleToInstantiableOperation;
template <typename... Operations>
struct OperationTupleToInstantiableOperation<OperationTuple<Operations...>> {
    FK_HD_STATIC auto value(const OperationTuple<Operations...>& t) { return detail::tuple_to_iop(t); }
};

// ---- batch reads ----------------------------------------------------------------------------------------------
enum class PlanePolicy { PROCESS_ALL = 0, CONDITIONAL_WITH_DEFAULT = 1 };

template <size_t BATCH, PlanePolicy PP, typename Operation, typename DefaultType>
struct BatchReadParams;
template <size_t BATCH, typename Operation, typename DefaultType>
struct BatchReadParams<BATCH, PlanePolicy::PROCESS_ALL, Operation, DefaultType> {
    OperationData<Operation> opData[BATCH];
    ActiveThreads activeThreads;
};
template <size_t BATCH, typename Operation, typename DefaultType>
struct BatchReadParams<BATCH, PlanePolicy::CONDITIONAL_WITH_DEFAULT, Operation, DefaultType> {
    OperationData<Operation> opData[BATCH];
    int usedPlanes;
    DefaultType default_value;
    ActiveThreads activeThreads;
};

template <size_t BATCH_, PlanePolicy PP_ = PlanePolicy::PROCESS_ALL, typename Operation_ = void, typename OutputType_ = NullType>
struct BatchRead;

namespace detail {
template <typename T, typename Alternative>
using NullTo = std::conditional_t<std::is_same_v<T, NullType>, Alternative, T>;
}

template <size_t BATCH_, PlanePolicy PP_, typename Operation_, typename OutputType_>
struct BatchRead {
private:
    using SelfType = BatchRead<BATCH_, PP_, Operation_, OutputType_>;

public:
    FK_STATIC_STRUCT(BatchRead, SelfType)
    static_assert(isAnyReadType<Operation_>, "The Operation is not of any Read type");
    using Operation = Operation_;
    static constexpr size_t BATCH = BATCH_;
    static constexpr PlanePolicy PP = PP_;
    using OutputType = detail::NullTo<typename Operation::OutputType, OutputType_>;
    using ReadDataType = detail::NullTo<typename Operation::ReadDataType, uchar>;
    using ParamsType = BatchReadParams<BATCH_, PP_, Operation_, OutputType>;
    using InstanceType = ReadType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Read<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;

    template <typename Op = Operation_>
    FK_HD_STATIC std::enable_if_t<isCompleteOperation<Op>, OutputType> exec(const Point& thread, const ParamsType& params) {
        if constexpr (PP_ == PlanePolicy::CONDITIONAL_WITH_DEFAULT) {
            if (params.usedPlanes <= thread.z) return params.default_value;
        }
        return Operation::exec(thread, params.opData[thread.z]);
    }
    template <typename Op = Operation_>
    FK_HD_STATIC std::enable_if_t<isCompleteOperation<Op>, OutputType> exec(const Point& thread, const OperationDataType& opData) {
        return exec(thread, opData.params);
    }
    FK_HD_STATIC uint num_elems_x(const Point& thread, const OperationDataType& opData) { return Operation::num_elems_x(thread, opData.params.opData[thread.z]); }
    FK_HD_STATIC uint num_elems_y(const Point& thread, const OperationDataType& opData) { return Operation::num_elems_y(thread, opData.params.opData[thread.z]); }
    FK_HD_STATIC uint num_elems_z(const Point&, const OperationDataType&) { return static_cast<uint>(BATCH_); }
    FK_HD_STATIC ActiveThreads getActiveThreads(const OperationDataType& opData) { return opData.params.activeThreads; }
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }
};

// Builder form: BatchRead<N, PP>::build(array of IOps [, usedPlanes, default]).
template <size_t BATCH_, PlanePolicy PP_>
struct BatchRead<BATCH_, PP_, void, NullType> {
    template <typename IOp>
    static inline constexpr auto build(const std::array<IOp, BATCH_>& iOps) {
        static_assert(PP_ == PlanePolicy::PROCESS_ALL, "CONDITIONAL_WITH_DEFAULT needs usedPlanes and a default value");
        static_assert(isAnyReadType<IOp>, "BatchRead is made of Read or ReadBack operations");
        using Op = typename IOp::Operation;
        using Batch = BatchRead<BATCH_, PlanePolicy::PROCESS_ALL, Op>;
        typename Batch::ParamsType params{};
        fill(params, iOps);
        return Batch::build(params);
    }
    template <typename IOp, typename DefaultValueType>
    static inline constexpr auto build(const std::array<IOp, BATCH_>& iOps, const int& usedPlanes, const DefaultValueType& defaultValue) {
        static_assert(isAnyReadType<IOp>, "BatchRead is made of Read or ReadBack operations");
        using Op = typename IOp::Operation;
        using Batch = BatchRead<BATCH_, PlanePolicy::CONDITIONAL_WITH_DEFAULT, Op, DefaultValueType>;
        typename Batch::ParamsType params{};
        fill(params, iOps);
        params.usedPlanes = usedPlanes;
        params.default_value = defaultValue;
        return Batch::build(params);
    }

    // A batch whose number of planes is known only at run time (this library's extension: the reference fixes it with
    // BATCH, batch_operations.h:153-208): the first `count` entries of a table of BATCH planes are filled in, and the
    // batch's thread grid has `count` planes.  box_w x box_h, when given, is the least extent of the thread grid: a caller
    // that launches one batch in several parts passes the largest width and height of the whole batch, so that every part
    // covers what the one batch would.
    template <typename IOp>
    static inline auto build_first(const IOp* iOps, size_t count, uint box_w = 0, uint box_h = 0) {
        static_assert(PP_ == PlanePolicy::PROCESS_ALL, "every plane of a run-time batch is processed");
        static_assert(isAnyReadType<IOp>, "BatchRead is made of Read or ReadBack operations");
        using Op = typename IOp::Operation;
        using Batch = BatchRead<BATCH_, PlanePolicy::PROCESS_ALL, Op>;
        typename Batch::ParamsType params{};
        count = count < BATCH_ ? count : BATCH_;
        uint max_w = box_w, max_h = box_h;
        for (size_t i = 0; i < count; ++i) {
            params.opData[i] = static_cast<const OperationData<Op>&>(iOps[i]);
            const uint w = Op::num_elems_x(Point(0, 0, 0), iOps[i]);
            const uint h = Op::num_elems_y(Point(0, 0, 0), iOps[i]);
            max_w = w > max_w ? w : max_w;
            max_h = h > max_h ? h : max_h;
        }
        params.activeThreads = ActiveThreads(max_w, max_h, static_cast<uint>(count));
        return Batch::build(params);
    }

private:
    template <typename Params, typename IOp>
    static inline constexpr void fill(Params& params, const std::array<IOp, BATCH_>& iOps) {
        using Op = typename IOp::Operation;
        uint max_w = 0, max_h = 0;
        for (size_t i = 0; i < BATCH_; ++i) {
            params.opData[i] = static_cast<const OperationData<Op>&>(iOps[i]);
            const uint w = Op::num_elems_x(Point(0, 0, 0), iOps[i]);
            const uint h = Op::num_elems_y(Point(0, 0, 0), iOps[i]);
            max_w = w > max_w ? w : max_w;
            max_h = h > max_h ? h : max_h;
        }
        params.activeThreads = ActiveThreads(max_w, max_h, static_cast<uint>(BATCH_));
    }
};

template <typename FirstOp, typename... ComputeOps>
template <size_t BATCH_N>
inline constexpr auto FusedOperation_<std::enable_if_t<isAnyReadType<FirstOp>>, FirstOp, ComputeOps...>::build(
    const std::array<InstantiableType, BATCH_N>& iOps) {
    return BatchRead<BATCH_N, PlanePolicy::PROCESS_ALL>::build(iOps);
}

struct BatchOperation {
    // The per-plane IOps of a batch read.
    template <typename BatchIOp>
    static inline constexpr auto toArray(const BatchIOp& batchIOp) {
        using Batch = typename BatchIOp::Operation;
        static_assert(isBatchOperation<Batch>, "The IOp passed as parameter is not a batch operation");
        using Op = typename Batch::Operation;
        std::array<Instantiable<Op>, Batch::BATCH> out{};
        for (size_t i = 0; i < Batch::BATCH; ++i) out[i] = toIOp<Op>(batchIOp.params.opData[i]);
        return out;
    }
    // Element-wise Operation::build over parallel arrays of build() arguments.
    template <typename Operation, size_t BATCH_N, typename First, typename... Arrays>
    static inline constexpr auto build_batch(const std::array<First, BATCH_N>& first, const Arrays&... arrays) {
        static_assert(((std::tuple_size_v<Arrays> == BATCH_N) && ...), "Not all arrays have the same size as BATCH");
        using IOp = decltype(Operation::build(first[0], arrays[0]...));
        std::array<IOp, BATCH_N> out{};
        for (size_t i = 0; i < BATCH_N; ++i) out[i] = Operation::build(first[i], arrays[i]...);
        return out;
    }
};

// build() overloads on arrays for read-like operations: `Self::build(std::array<...>, ...)` makes one plane per element
// (batch_operations.h:380-504).  An operation opts in by deriving from this.
namespace detail {
template <typename First, typename Self, typename = void>
struct IsIOpOf : std::false_type {};
template <typename First, typename Self>
struct IsIOpOf<First, Self, std::void_t<typename First::Operation>> : std::is_same<typename First::Operation, Self> {};
} // namespace detail

template <typename Self>
struct BatchBuilders {
    template <size_t BATCH_N, typename First, typename... Arrays>
    static inline constexpr auto build_batch(const std::array<First, BATCH_N>& first, const Arrays&... arrays) {
        return BatchOperation::build_batch<Self>(first, arrays...);
    }
    template <size_t BATCH_N, typename First, typename... Arrays>
    static inline constexpr auto build(const std::array<First, BATCH_N>& first, const Arrays&... arrays) {
        if constexpr (sizeof...(Arrays) == 0 && detail::IsIOpOf<First, Self>::value) {
            return BatchRead<BATCH_N, PlanePolicy::PROCESS_ALL>::build(first);
        } else {
            return BatchRead<BATCH_N, PlanePolicy::PROCESS_ALL>::build(BatchOperation::build_batch<Self>(first, arrays...));
        }
    }
    template <size_t BATCH_N, typename DefaultValueType, typename First, typename... Arrays>
    static inline constexpr auto build(const int& usedPlanes, const DefaultValueType& defaultValue,
                                       const std::array<First, BATCH_N>& first, const Arrays&... arrays) {
        if constexpr (sizeof...(Arrays) == 0 && detail::IsIOpOf<First, Self>::value) {
            return BatchRead<BATCH_N, PlanePolicy::CONDITIONAL_WITH_DEFAULT>::build(first, usedPlanes, defaultValue);
        } else {
            return BatchRead<BATCH_N, PlanePolicy::CONDITIONAL_WITH_DEFAULT>::build(
                BatchOperation::build_batch<Self>(first, arrays...), usedPlanes, defaultValue);
        }
    }
};

// ---- batch writes ---------------------------------------------------------------------------------------------
// BATCH writes of one kind behind one Write operation: plane thread.z goes to its own destination
// (operation_model/batch_operations.h:320-377).  The parameters are the plain array of the per-plane parameters.
template <size_t BATCH_, typename Operation_ = void>
struct BatchWrite {
private:
    using SelfType = BatchWrite<BATCH_, Operation_>;

public:
    FK_STATIC_STRUCT(BatchWrite, SelfType)
    static_assert(isWriteType<Operation_>, "The Operation is not of Write type");
    using Operation = Operation_;
    static constexpr size_t BATCH = BATCH_;
    using InputType = typename Operation::InputType;
    using ParamsType = typename Operation::ParamsType[BATCH_];
    using WriteDataType = typename Operation::WriteDataType;
    using InstanceType = WriteType;
    using OperationDataType = OperationData<SelfType>;
    using InstantiableType = Write<SelfType>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = false;

    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const ParamsType& params) { Operation::exec(thread, input, params[thread.z]); }
    FK_HD_STATIC void exec(const Point& thread, const InputType& input, const OperationDataType& opData) { exec(thread, input, opData.params); }
    FK_HD_STATIC uint num_elems_x(const Point& thread, const OperationDataType& opData) { return Operation::num_elems_x(thread, { opData.params[thread.z] }); }
    FK_HD_STATIC uint pitch(const Point& thread, const OperationDataType& opData) { return Operation::pitch(thread, { opData.params[thread.z] }); }
    template <typename IOp>
    static inline constexpr std::enable_if_t<isWriteType<IOp>, InstantiableType> build(const std::array<IOp, BATCH_>& iOps) {
        static_assert(std::is_same_v<typename IOp::Operation, Operation_>, "The IOps in the array are of another operation");
        InstantiableType out{};
        for (size_t i = 0; i < BATCH_; ++i) out.params[i] = iOps[i].params;
        return out;
    }
    template <typename First, typename... Arrays>
    static inline constexpr std::enable_if_t<!isWriteType<First>, InstantiableType> build(const std::array<First, BATCH_>& first, const Arrays&... arrays) {
        return build(Operation::build_batch(first, arrays...));
    }
};
// Builder form: BatchWrite<N>::build(array of Write IOps).
template <size_t BATCH_>
struct BatchWrite<BATCH_, void> {
    template <typename IOp>
    static inline constexpr auto build(const std::array<IOp, BATCH_>& iOps) {
        return BatchWrite<BATCH_, typename IOp::Operation>::build(iOps);
    }
};

// ---- Fuser ----------------------------------------------------------------------------------------------------
namespace detail {
template <typename O, typename I>
FK_HD_CNST O cast_channels(const I& v) {
    if constexpr (std::is_same_v<I, O>) {
        return v;
    } else if constexpr (!validCUDAVec<O>) {
        return static_cast<O>(vget<0>(v));
    } else if constexpr (cn<O> == 1) {
        return make_<O>(vget<0>(v));
    } else if constexpr (cn<O> == 2) {
        return make_<O>(vget<0>(v), vget<1>(v));
    } else if constexpr (cn<O> == 3) {
        return make_<O>(vget<0>(v), vget<1>(v), vget<2>(v));
    } else {
        return make_<O>(vget<0>(v), vget<1>(v), vget<2>(v), vget<3>(v));
    }
}
} // namespace detail

struct Fuser {
    template <typename FirstIOp, typename SecondIOp>
    static inline constexpr auto fuse(const FirstIOp& first, const SecondIOp& second) {
        using SelfOp = typename FirstIOp::Operation;
        using ContOp = typename SecondIOp::Operation;
        static_assert(!isReadType<SecondIOp> || isBatchOperation<ContOp>,
                      "ReadOperation as continuation is not allowed. It has to be a ReadBackOperation.");
        if constexpr (!isBatchOperation<SelfOp> && !isBatchOperation<ContOp>) {
            return fusePlain(first, second);
        } else {
            return fuseBatch(first, second);
        }
    }
    template <typename FirstIOp, typename SecondIOp, typename... RestIOps>
    static inline constexpr auto fuse(const FirstIOp& first, const SecondIOp& second, const RestIOps&... rest) {
        return fuse(fuse(first, second), rest...);
    }

private:
    template <typename SelfIOp, typename ContIOp>
    static inline constexpr auto fusePlain(const SelfIOp& self, const ContIOp& cont) {
        if constexpr (isReadBackType<ContIOp>) {
            // the continuation is a ReadBack builder waiting for its back read: complete it with what came before
            return ContIOp::Operation::build(self, cont);
        } else {
            return detail::tuple_to_iop(operation_tuple_cat(detail::iop_to_tuple(self), detail::iop_to_tuple(cont)));
        }
    }
    template <size_t I, typename IOp>
    static inline constexpr auto planeOf(const IOp& iOp) {
        if constexpr (isBatchOperation<typename IOp::Operation>) {
            return toIOp<typename IOp::Operation::Operation>(iOp.params.opData[I]);
        } else {
            return iOp;
        }
    }
    template <typename SelfIOp, typename ContIOp, size_t... Idx>
    static inline constexpr auto fusePlanes(const SelfIOp& self, const ContIOp& cont, std::index_sequence<Idx...>) {
        using Fused = decltype(fusePlain(planeOf<0>(self), planeOf<0>(cont)));
        return std::array<Fused, sizeof...(Idx)>{ fusePlain(planeOf<Idx>(self), planeOf<Idx>(cont))... };
    }
    template <typename Op>
    static constexpr PlanePolicy policyOf() {
        if constexpr (isBatchOperation<Op>) return Op::PP;
        else return PlanePolicy::PROCESS_ALL;
    }
    template <typename Op>
    static constexpr size_t batchOf() {
        if constexpr (isBatchOperation<Op>) return static_cast<size_t>(Op::BATCH);
        else return 0;
    }
    template <typename SelfIOp, typename ContIOp>
    static inline constexpr auto fuseBatch(const SelfIOp& self, const ContIOp& cont) {
        using SelfOp = typename SelfIOp::Operation;
        using ContOp = typename ContIOp::Operation;
        constexpr size_t NS = batchOf<SelfOp>(), NC = batchOf<ContOp>();
        static_assert(NS == 0 || NC == 0 || NS == NC, "Fusing two batch operations of different BATCH size is not allowed.");
        constexpr size_t N = NS != 0 ? NS : NC;
        if constexpr (NC != 0) {
            static_assert(isReadBackType<typename ContOp::Operation>,
                          "ReadOperation as continuation is not allowed. It has to be a ReadBackOperation.");
        }
        const auto planes = fusePlanes(self, cont, std::make_index_sequence<N>{});
        using PlaneIOp = typename decltype(planes)::value_type;
        using NewOutput = typename PlaneIOp::Operation::OutputType;
        if constexpr (policyOf<ContOp>() == PlanePolicy::CONDITIONAL_WITH_DEFAULT) {
            return BatchRead<N, PlanePolicy::CONDITIONAL_WITH_DEFAULT>::build(
                planes, cont.params.usedPlanes, detail::cast_channels<NewOutput>(cont.params.default_value));
        } else if constexpr (policyOf<SelfOp>() == PlanePolicy::CONDITIONAL_WITH_DEFAULT) {
            if constexpr (isComputeType<ContIOp>) {
                // the default value of the unused planes flows through the compute operation like any other value, as it
                // does when the operation follows the batch read as a separate argument of executeOperations
                return BatchRead<N, PlanePolicy::CONDITIONAL_WITH_DEFAULT>::build(
                    planes, self.params.usedPlanes,
                    detail::cast_channels<NewOutput>(compute(detail::cast_channels<GetInputType_t<ContIOp>>(self.params.default_value), cont)));
            } else {
                return BatchRead<N, PlanePolicy::CONDITIONAL_WITH_DEFAULT>::build(
                    planes, self.params.usedPlanes, detail::cast_channels<NewOutput>(self.params.default_value));
            }
        } else {
            return BatchRead<N, PlanePolicy::PROCESS_ALL>::build(planes);
        }
    }
};

template <typename... IOps>
inline constexpr auto fuse(const IOps&... iOps) {
    return Fuser::fuse(iOps...);
}

} // namespace fk
#endif
