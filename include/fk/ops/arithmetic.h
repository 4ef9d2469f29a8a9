// Element-wise compute operations: Add/Sub/Mul/Div, Cast, SaturateCast, VectorReorder, Discard, Max/Min.
// Semantics follow the reference's algorithms/basic_ops/arithmetic.h:22-88, cast.h:22-33 + cast_base.h:19-31,
// algorithms/image_processing/saturate.h:27-67 (+ cxp::round, core/constexpr_libs/constexpr_cmath.h:119-130),
// algorithms/basic_ops/cuda_vector.h:22-62 and logical.h (Max/Min).
#ifndef FK_OPS_ARITHMETIC_H
#define FK_OPS_ARITHMETIC_H

#include <limits>

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
FK_ARITHMETIC_OPERATION(Add, +)
FK_ARITHMETIC_OPERATION(Sub, -)
FK_ARITHMETIC_OPERATION(Mul, *)
FK_ARITHMETIC_OPERATION(Div, /)
#undef FK_ARITHMETIC_OPERATION

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

namespace cxp {
// Half away from zero through an int cast (constexpr_cmath.h:119-130).
template <typename T>
FK_HD_CNST T round(T x) {
    static_assert(std::is_floating_point_v<T>, "Input must be a floating-point type");
    if (x != x || x == std::numeric_limits<T>::infinity() || x == -std::numeric_limits<T>::infinity()) return x;
    return (x > T(0)) ? static_cast<T>(static_cast<int>(x + T(0.5))) : static_cast<T>(static_cast<int>(x - T(0.5)));
}
template <typename T>
FK_HD_CNST T max(const T& a, const T& b) { return a >= b ? a : b; }
template <typename T>
FK_HD_CNST T min(const T& a, const T& b) { return a <= b ? a : b; }
// Sign-safe comparisons between arithmetic types (constexpr_cmath.h:75-117).
template <typename T, typename U>
FK_HD_CNST bool cmp_less(const T& t, const U& u) {
    if constexpr (std::is_floating_point_v<T> || std::is_floating_point_v<U>) {
        return t < u;
    } else if constexpr (std::is_signed_v<T> == std::is_signed_v<U>) {
        return t < u;
    } else if constexpr (std::is_signed_v<T>) {
        return t < 0 || static_cast<std::make_unsigned_t<T>>(t) < u;
    } else {
        return u >= 0 && t < static_cast<std::make_unsigned_t<U>>(u);
    }
}
template <typename T, typename U>
FK_HD_CNST bool cmp_greater(const T& t, const U& u) { return cmp_less(u, t); }
} // namespace cxp

template <typename T>
constexpr T maxValue = std::numeric_limits<T>::max();
template <typename T>
constexpr T minValue = std::numeric_limits<T>::lowest();

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
            if constexpr (std::is_same_v<I, float>) clamped = __builtin_fmaxf(__builtin_fminf(input, above), below);
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

template <typename I, typename P = I, typename O = I>
struct Max {
private:
    using SelfType = Max<I, P, O>;

public:
    FK_BINARY_OPERATION(Max, I, P, O)
    FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) { return static_cast<O>(input >= params ? input : params); }
};
template <typename I, typename P = I, typename O = I>
struct Min {
private:
    using SelfType = Min<I, P, O>;

public:
    FK_BINARY_OPERATION(Min, I, P, O)
    FK_HD_STATIC OutputType exec(const InputType& input, const ParamsType& params) { return static_cast<O>(input <= params ? input : params); }
};

} // namespace fk
#endif
