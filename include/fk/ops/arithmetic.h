// Element-wise compute operations: Add/Sub/Mul/Div, Cast, SaturateCast, VectorReorder, Discard, Max/Min.
// Semantics follow the reference's algorithms/basic_ops/arithmetic.h:22-88, cast.h:22-33 + cast_base.h:19-31,
// algorithms/image_processing/saturate.h:27-67 (+ cxp::round, core/constexpr_libs/constexpr_cmath.h:119-130),
// algorithms/basic_ops/cuda_vector.h:22-62 and logical.h (Max/Min).
#ifndef FK_OPS_ARITHMETIC_H
#define FK_OPS_ARITHMETIC_H

#include <limits>

#include "fk/core/constexpr_cmath.h"
#include "fk/core/operation_model.h"

namespace fk {

#define FK_UNARY_OPERATION(SELF, I, O)                                                                                 \
    FK_STATIC_STRUCT(SELF, SelfType)                                                                                   \
    using InputType = I;                                                                                               \
    using OutputType = O;                                                                                              \
    using InstanceType = UnaryType;                                                                                    \
    using InstantiableType = Unary<SelfType>;                                                                          \
    static constexpr bool IS_FUSED_OP = false;                                                                         \
    FK_HD_STATIC InstantiableType build() { return InstantiableType{}; }

#define FK_BINARY_OPERATION(SELF, I, P, O)                                                                             \
    FK_STATIC_STRUCT(SELF, SelfType)                                                                                   \
    using InputType = I;                                                                                               \
    using ParamsType = P;                                                                                              \
    using OutputType = O;                                                                                              \
    using InstanceType = BinaryType;                                                                                   \
    using OperationDataType = OperationData<SelfType>;                                                                 \
    using InstantiableType = Binary<SelfType>;                                                                         \
    static constexpr bool IS_FUSED_OP = false;                                                                         \
    FK_HD_STATIC OutputType exec(const InputType& input, const OperationDataType& opData) { return exec(input, opData.params); } \
    FK_HD_STATIC InstantiableType build(const ParamsType& params) { return InstantiableType{ { params } }; }           \
    FK_HD_STATIC InstantiableType build(const OperationDataType& opData) { return InstantiableType{ opData }; }

#define FK_ARITHMETIC_OPERATION(NAME, OP)                                                                              \
    template <typename I, typename P = I, typename O = I>                                                              \
    struct NAME {                                                                                                      \
    private:                                                                                                           \
        using SelfType = NAME<I, P, O>;                                                                                \
                                                                                                                       \
    public:                                                                                                            \
        FK_BINARY_OPERATION(NAME, I, P, O)                                                                             \
        FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) {                               \
            return detail::cast_channels<O>(input OP params);                                                          \
        }                                                                                                              \
    };
FK_ARITHMETIC_OPERATION(Sub, -)
FK_ARITHMETIC_OPERATION(Mul, *)
FK_ARITHMETIC_OPERATION(Div, /)
#undef FK_ARITHMETIC_OPERATION

// Add has two forms: Binary (input + parameter), and Unary over a Tuple of both operands (basic_ops/arithmetic.h:21-48).
template <typename I1, typename I2 = I1, typename O = I1, typename IT = BinaryType>
struct Add;
template <typename I, typename P, typename O>
struct Add<I, P, O, BinaryType> {
private:
    using SelfType = Add<I, P, O, BinaryType>;

public:
    FK_BINARY_OPERATION(Add, I, P, O)
    FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) { return detail::cast_channels<O>(input + params); }
};
template <typename I1, typename I2, typename O>
struct Add<I1, I2, O, UnaryType> {
private:
    using SelfType = Add<I1, I2, O, UnaryType>;
    using Operands = Tuple<I1, I2>;

public:
    FK_UNARY_OPERATION(Add, Operands, O)
    FK_HD_STATIC OutputType exec(const InputType& input) { return detail::cast_channels<O>(get<0>(input) + get<1>(input)); }
};

// static_cast per channel
template <typename I, typename O>
struct Cast {
private:
    using SelfType = Cast<I, O>;

public:
    FK_UNARY_OPERATION(Cast, I, O)
    static_assert(cn<I> == cn<O>, "Cast keeps the number of channels");
    FK_HD_STATIC OutputType exec(const InputType& input) { return detail::cast_channels<O>(input); }
};


template <typename T>
constexpr T maxValue = make_set<T>(std::numeric_limits<VBase<T>>::max()); // every channel, for a vector type
template <typename T>
constexpr T minValue = make_set<T>(std::numeric_limits<VBase<T>>::lowest());

template <typename I, typename O>
struct SaturateCastBase {
private:
    using SelfType = SaturateCastBase<I, O>;

public:
    FK_UNARY_OPERATION(SaturateCastBase, I, O)
    FK_HD_STATIC OutputType exec(const InputType& input) {
        constexpr O hi = maxValue<O>;
        constexpr O lo = minValue<O>;
        if constexpr (std::is_floating_point_v<I> && std::is_integral_v<O> && sizeof(O) < sizeof(int)) {
            // The same value as the general form below for every finite input, written without branches: clamp first
            // (the limits are integers, so rounding leaves them alone), then round half away from zero through int.
            const I above = static_cast<I>(hi), below = static_cast<I>(lo);
            I clamped{};
            if constexpr (std::is_same_v<I, float>) {
#if defined(__HIP_DEVICE_COMPILE__)
                // the median of (input, lowest, highest) is the clamped value, in one instruction
                if (!__builtin_is_constant_evaluated()) clamped = __builtin_amdgcn_fmed3f(input, below, above);
                else
#endif
                    clamped = __builtin_fmaxf(__builtin_fminf(input, above), below);
            }
            else clamped = static_cast<I>(__builtin_fmax(__builtin_fmin(static_cast<double>(input), static_cast<double>(above)), static_cast<double>(below)));
            if constexpr (std::is_unsigned_v<O>) {
                return static_cast<O>(static_cast<int>(clamped + I(0.5))); // clamped >= 0, and (int)(0 - 0.5) == (int)(0 + 0.5)
            } else {
                return static_cast<O>(static_cast<int>(clamped + (clamped > I(0) ? I(0.5) : I(-0.5))));
            }
        } else {
            if (cxp::cmp_greater(input, hi)) return hi;
            if (cxp::cmp_less(input, lo)) return lo;
            if constexpr (std::is_floating_point_v<I> && std::is_integral_v<O>) {
                return static_cast<O>(cxp::round(input));
            } else {
                return static_cast<O>(input);
            }
        }
    }
};

// Clamp to the output range; float -> integer rounds half away from zero.
template <typename I, typename O>
struct SaturateCast {
private:
    using SelfType = SaturateCast<I, O>;
    using Base = SaturateCastBase<VBase<I>, VBase<O>>;

public:
    FK_UNARY_OPERATION(SaturateCast, I, O)
    static_assert(cn<I> == cn<O>, "SaturateCast keeps the number of channels");
    FK_HD_STATIC OutputType exec(const InputType& input) {
        if constexpr (!validCUDAVec<I>) {
            return Base::exec(input);
        } else if constexpr (cn<I> == 1) {
            return O{ Base::exec(input.x) };
        } else if constexpr (cn<I> == 2) {
            return O{ Base::exec(input.x), Base::exec(input.y) };
        } else if constexpr (cn<I> == 3) {
            return O{ Base::exec(input.x), Base::exec(input.y), Base::exec(input.z) };
        } else {
            return O{ Base::exec(input.x), Base::exec(input.y), Base::exec(input.z), Base::exec(input.w) };
        }
    }
};

// Channel permutation: output channel k takes input channel IDX[k].
template <typename T, int... IDX>
struct VectorReorder {
private:
    using SelfType = VectorReorder<T, IDX...>;

public:
    FK_UNARY_OPERATION(VectorReorder, T, T)
    static_assert(validCUDAVec<T> && cn<T> >= 2, "VectorReorder needs a vector type with two or more channels");
    static_assert(sizeof...(IDX) == cn<T>, "One index per channel");
    FK_HD_STATIC OutputType exec(const InputType& input) { return T{ vget<IDX>(input)... }; }
};

// Drops trailing channels.
template <typename I, typename O>
struct Discard {
private:
    using SelfType = Discard<I, O>;

public:
    FK_UNARY_OPERATION(Discard, I, O)
    static_assert(cn<I> > cn<O>, "Output type should at least have one channel less");
    static_assert(std::is_same_v<VBase<I>, VBase<O>>, "Base types should be the same");
    FK_HD_STATIC OutputType exec(const InputType& input) { return detail::cast_channels<O>(input); }
};

// ---- per-channel application of a scalar operation (operation_model/vector_operations.h:23-189) -----------------
// UnaryV<Op, I, O>: O{ Op(i.x), Op(i.y), ... }; with a Tuple<I1, I2> input Op gets Tuple{ i1.x, i2.x } per channel, where
// a scalar second operand is used for every channel.  BinaryV<Op, I, P, O>: O{ Op(i.x, p.x), ... }, same rule for P.
namespace detail {
template <typename In, typename Out>
constexpr bool both_vectors_or_none = validCUDAVec<In> == validCUDAVec<Out>;
}
template <typename Operation, typename I, typename O, typename = void>
struct UnaryV {
private:
    using SelfType = UnaryV<Operation, I, O, void>;
    template <int... K>
    FK_HD_STATIC O channels(const I& input, std::integer_sequence<int, K...>) {
        if constexpr (validCUDAVec<O>) {
            return O{ Operation::exec(vget<K>(input))... };
        } else {
            return Operation::exec(input);
        }
    }

public:
    FK_STATIC_STRUCT(UnaryV, SelfType)
    using InputType = I;
    using OutputType = O;
    using InstanceType = UnaryType;
    static_assert(cn<I> == cn<O>, "UnaryV requires the same number of channels for input and output types.");
    static_assert(detail::both_vectors_or_none<I, O>, "UnaryV requires input and output types to be both vector types or none.");
    FK_HD_STATIC OutputType exec(const InputType& input) { return channels(input, std::make_integer_sequence<int, cn<I>>{}); }
};
template <typename Operation, typename I, typename O>
struct UnaryV<Operation, I, O, std::enable_if_t<isTuple_v<I>>> {
private:
    using SelfType = UnaryV<Operation, I, O, void>;
    using I1 = get_t<0, I>;
    using I2 = get_t<1, I>;
    template <int... K>
    FK_HD_STATIC O channels(const I1& a, const I2& b, std::integer_sequence<int, K...>) {
        using Pair = typename Operation::InputType;
        if constexpr (validCUDAVec<O>) {
            return O{ Operation::exec(Pair{ vget<K>(a), vget<K>(b) })... };
        } else {
            return Operation::exec(Pair{ a, b });
        }
    }

public:
    FK_STATIC_STRUCT(UnaryV, SelfType)
    using InputType = I;
    using OutputType = O;
    using InstanceType = UnaryType;
    static_assert(cn<I1> == cn<O>, "UnaryV requires the same number of channels for input and output types.");
    static_assert(detail::both_vectors_or_none<I1, O>, "UnaryV requires input and output types to be both vector types or none.");
    FK_HD_STATIC OutputType exec(const InputType& input) { return channels(get<0>(input), get<1>(input), std::make_integer_sequence<int, cn<I1>>{}); }
};
template <typename Operation, typename I, typename P = I, typename O = I>
struct BinaryV {
private:
    using SelfType = BinaryV<Operation, I, P, O>;
    template <int... K>
    FK_HD_STATIC O channels(const I& input, const P& params, std::integer_sequence<int, K...>) {
        if constexpr (validCUDAVec<O>) {
            return O{ Operation::exec(vget<K>(input), vget<K>(params))... };
        } else {
            return Operation::exec(input, params);
        }
    }

public:
    FK_STATIC_STRUCT(BinaryV, SelfType)
    using InputType = I;
    using ParamsType = P;
    using OutputType = O;
    using InstanceType = BinaryType;
    using OperationDataType = OperationData<SelfType>;
    static_assert(cn<I> == cn<O>, "BinaryV requires the same number of channels for input and output types.");
    static_assert(detail::both_vectors_or_none<I, O>, "BinaryV requires input and output types to be both vector types or none.");
    FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) { return channels(input, params, std::make_integer_sequence<int, cn<I>>{}); }
    FK_HD_STATIC OutputType exec(const InputType& input, const OperationDataType& opData) { return exec(input, opData.params); }
};

// ---- Max / Min (basic_ops/logical.h:84-194): per channel, on a tie the parameter; Binary and Tuple-input Unary forms --
#define FK_EXTREME_OPERATION(NAME, BASE, PICK)                                                                         \
    template <typename I, typename P = I, typename O = I, typename IT = BinaryType>                                    \
    struct BASE {                                                                                                      \
    private:                                                                                                           \
        using SelfType = BASE<I, P, O, BinaryType>;                                                                    \
                                                                                                                       \
    public:                                                                                                            \
        FK_BINARY_OPERATION(BASE, I, P, O)                                                                             \
        static_assert(!validCUDAVec<I> && !validCUDAVec<P> && !validCUDAVec<O>, #BASE " works on scalars.");           \
        FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) { return cxp::PICK(input, params); } \
    };                                                                                                                 \
    template <typename I, typename P, typename O>                                                                      \
    struct BASE<I, P, O, UnaryType> {                                                                                  \
    private:                                                                                                           \
        using SelfType = BASE<I, P, O, UnaryType>;                                                                     \
        using Operands = Tuple<I, P>;                                                                                  \
                                                                                                                       \
    public:                                                                                                            \
        FK_UNARY_OPERATION(BASE, Operands, O)                                                                          \
        static_assert(!validCUDAVec<I> && !validCUDAVec<P> && !validCUDAVec<O>, #BASE " works on scalars.");           \
        FK_HD_STATIC OutputType exec(const InputType& input) { return cxp::PICK(get<0>(input), get<1>(input)); }       \
    };                                                                                                                 \
    template <typename I, typename P = I, typename O = I, typename IT = BinaryType>                                    \
    struct NAME {                                                                                                      \
    private:                                                                                                           \
        using SelfType = NAME<I, P, O, BinaryType>;                                                                    \
                                                                                                                       \
    public:                                                                                                            \
        FK_BINARY_OPERATION(NAME, I, P, O)                                                                             \
        FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) {                               \
            return BinaryV<BASE<VBase<I>, VBase<P>, VBase<O>>, I, P, O>::exec(input, params);                          \
        }                                                                                                              \
    };                                                                                                                 \
    template <typename I, typename P, typename O>                                                                      \
    struct NAME<I, P, O, UnaryType> {                                                                                  \
    private:                                                                                                           \
        using SelfType = NAME<I, P, O, UnaryType>;                                                                     \
        using Operands = Tuple<I, P>;                                                                                  \
                                                                                                                       \
    public:                                                                                                            \
        FK_UNARY_OPERATION(NAME, Operands, O)                                                                          \
        FK_HD_STATIC OutputType exec(const InputType& input) {                                                         \
            return UnaryV<BASE<VBase<I>, VBase<P>, VBase<O>, UnaryType>, Operands, O>::exec(input);                    \
        }                                                                                                              \
    };
FK_EXTREME_OPERATION(Max, MaxBase, max)
FK_EXTREME_OPERATION(Min, MinBase, min)
#undef FK_EXTREME_OPERATION

// All channels of both operands equal (basic_ops/logical.h:196-223).
template <typename I1, typename I2 = I1>
struct Equal {
private:
    using SelfType = Equal<I1, I2>;
    using Operands = Tuple<I1, I2>;

public:
    FK_UNARY_OPERATION(Equal, Operands, bool)
    FK_HD_STATIC OutputType exec(const InputType& input) {
        if constexpr (validCUDAVec<I1>) {
            return Bool::vAnd(get<0>(input) == get<1>(input));
        } else {
            return get<0>(input) == get<1>(input);
        }
    }
};

// ---- more vector operations (basic_ops/cuda_vector.h:75-176) ---------------------------------------------------------
// Channel permutation chosen at run time: output channel k takes input channel params[k].
template <typename T>
struct VectorReorderRT {
private:
    using SelfType = VectorReorderRT<T>;
    using Order = VectorType_t<int, cn<T>>;
    template <int... K>
    FK_HD_STATIC T pick(const T& input, const Order& order, std::integer_sequence<int, K...>) {
        const VBase<T> channel[cn<T>]{ vget<K>(input)... };
        return T{ channel[vget<K>(order)]... };
    }

public:
    FK_BINARY_OPERATION(VectorReorderRT, T, Order, T)
    static_assert(validCUDAVec<T> && cn<T> >= 2, "VectorReorderRT needs a vector type with two or more channels");
    FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) { return pick(input, params, std::make_integer_sequence<int, cn<T>>{}); }
};

// Folds the channels from left to right with a two-operand operation: Op(Op(x, y), z)...  The operation is Binary, or Unary
// over a Tuple of both operands.
template <typename T, typename Operation>
struct VectorReduce {
private:
    using SelfType = VectorReduce<T, Operation>;
    using Result = typename Operation::OutputType;
    template <typename A, typename B>
    FK_HD_STATIC Result combine(const A& a, const B& b) {
        if constexpr (isUnaryType<Operation>) {
            using Pair = typename Operation::InputType;
            return Operation::exec(Pair{ static_cast<get_t<0, Pair>>(a), static_cast<get_t<1, Pair>>(b) });
        } else {
            return Operation::exec(a, b);
        }
    }

public:
    FK_UNARY_OPERATION(VectorReduce, T, Result)
    FK_HD_STATIC OutputType exec(const InputType& input) {
        if constexpr (cn<T> == 1) {
            return vget<0>(input);
        } else if constexpr (cn<T> == 2) {
            return combine(input.x, input.y);
        } else if constexpr (cn<T> == 3) {
            return combine(combine(input.x, input.y), input.z);
        } else {
            return combine(combine(combine(input.x, input.y), input.z), input.w);
        }
    }
};

// The channels of a bool vector folded with equality, as the reference defines it (cuda_vector.h:157-169): true for an
// all-true vector, and the fold (x == y) == z ... for any other.
template <typename T>
struct VectorAnd {
private:
    using SelfType = VectorAnd<T>;

public:
    FK_UNARY_OPERATION(VectorAnd, T, bool)
    FK_HD_STATIC OutputType exec(const InputType& input) { return VectorReduce<T, Equal<bool, bool>>::exec(input); }
};
template <typename T>
FK_HD_CNST bool vecAnd(const T& value) {
    return VectorAnd<T>::exec(value);
}

// Appends the parameter as one more channel.
template <typename I, typename O>
struct AddLast {
private:
    using SelfType = AddLast<I, O>;
    using Channel = VBase<I>;
    template <int... K>
    FK_HD_STATIC O append(const I& input, const Channel& last, std::integer_sequence<int, K...>) {
        return O{ vget<K>(input)..., last };
    }

public:
    FK_BINARY_OPERATION(AddLast, I, Channel, O)
    static_assert(cn<I> == cn<O> - 1, "Output type should have one channel more");
    static_assert(std::is_same_v<VBase<I>, VBase<O>>, "Base types should be the same");
    FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) { return append(input, params, std::make_integer_sequence<int, cn<I>>{}); }
};

} // namespace fk
#endif
