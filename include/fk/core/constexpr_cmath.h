// Math helpers that are usable in constant expressions and in device code alike.
//
// Same names and results as the reference's core/constexpr_libs/constexpr_cmath.h:23-181: limits as variable templates,
// isnan/isinf without library calls, comparisons between integers of different signedness that never convert a negative
// value to unsigned, round half away from zero through an int cast, max/min over any number of equal-typed values (on a
// tie, or on an unordered comparison, the later argument wins), and abs.
#ifndef FK_CORE_CONSTEXPR_CMATH_H
#define FK_CORE_CONSTEXPR_CMATH_H

#include <limits>
#include <type_traits>

#include "fk/core/utils.h"

namespace fk {
namespace cxp {
template <typename T>
constexpr T minValue = std::numeric_limits<T>::lowest();
template <typename T>
constexpr T maxValue = std::numeric_limits<T>::max();
template <typename T>
constexpr T smallestPositiveValue = std::is_floating_point_v<T> ? std::numeric_limits<T>::min() : static_cast<T>(1);

// NaN is the only value that differs from itself; an infinity is the only non-zero value that doubling leaves unchanged.
template <typename T>
FK_HD_CNST bool isnan(T x) {
    return !(x == x);
}
template <typename T>
FK_HD_CNST bool isinf(T x) {
    return !isnan(x) && x != T(0) && x + x == x;
}

namespace detail {
// Integers of different signedness are compared by sign first and, when both are non-negative, as unsigned magnitudes;
// every other pair of arithmetic types compares as the language compares them.
template <typename T, typename U>
constexpr bool mixed_signs = std::is_integral_v<T> && std::is_integral_v<U> && (std::is_signed_v<T> != std::is_signed_v<U>);
template <typename T>
FK_HD_CNST bool below_zero(const T& v) {
    if constexpr (std::is_signed_v<T>) {
        return v < T(0);
    } else {
        return false;
    }
}
template <typename T>
FK_HD_CNST auto magnitude(const T& v) { // of a value that is not below zero
    return static_cast<std::make_unsigned_t<T>>(v);
}
template <typename T, typename U>
constexpr bool comparable = std::is_fundamental_v<T> && std::is_fundamental_v<U> && !std::is_same_v<T, bool> && !std::is_same_v<U, bool>;
} // namespace detail

template <typename T, typename U>
FK_HD_CNST bool cmp_less(const T& t, const U& u) {
    static_assert(detail::comparable<T, U>, "Both parameters must be fundamental types other than bool");
    if constexpr (detail::mixed_signs<T, U>) {
        if (detail::below_zero(t) != detail::below_zero(u)) return detail::below_zero(t);
        return detail::magnitude(t) < detail::magnitude(u); // both are non-negative here: one of them is unsigned
    } else {
        return t < u;
    }
}
template <typename T, typename U>
FK_HD_CNST bool cmp_equal(const T& t, const U& u) {
    static_assert(detail::comparable<T, U>, "Both parameters must be fundamental types other than bool");
    if constexpr (detail::mixed_signs<T, U>) {
        return !detail::below_zero(t) && !detail::below_zero(u) && detail::magnitude(t) == detail::magnitude(u);
    } else {
        return t == u;
    }
}
template <typename T, typename U>
FK_HD_CNST bool cmp_not_equal(const T& t, const U& u) {
    return !cmp_equal(t, u);
}
template <typename T, typename U>
FK_HD_CNST bool cmp_greater(const T& t, const U& u) {
    return cmp_less(u, t);
}
template <typename T, typename U>
FK_HD_CNST bool cmp_less_equal(const T& t, const U& u) {
    return !cmp_less(u, t);
}
template <typename T, typename U>
FK_HD_CNST bool cmp_greater_equal(const T& t, const U& u) {
    return !cmp_less(t, u);
}

// Half away from zero through an int cast (so only for magnitudes an int holds); NaN and the infinities pass through.
template <typename T>
FK_HD_CNST T round(T x) {
    static_assert(std::is_floating_point_v<T>, "Input must be a floating-point type");
    if (isnan(x) || isinf(x)) return x;
    const T half = x > T(0) ? T(0.5) : T(-0.5);
    return static_cast<T>(static_cast<int>(x + half));
}

namespace detail {
// folds from the right: the later argument wins a tie
template <bool LARGEST, typename T>
FK_HD_CNST T extreme(const T& only) {
    return only;
}
template <bool LARGEST, typename T, typename... Ts>
FK_HD_CNST T extreme(const T& first, const Ts&... rest) {
    const T later = extreme<LARGEST>(rest...);
    if constexpr (LARGEST) {
        return first >= later ? first : later;
    } else {
        return first <= later ? first : later;
    }
}
} // namespace detail
template <typename T, typename... Ts>
FK_HD_CNST T max(const T& first, const Ts&... rest) {
    static_assert((std::is_same_v<T, Ts> && ...), "All types must be the same");
    return detail::extreme<true>(first, rest...);
}
template <typename T, typename... Ts>
FK_HD_CNST T min(const T& first, const Ts&... rest) {
    static_assert((std::is_same_v<T, Ts> && ...), "All types must be the same");
    return detail::extreme<false>(first, rest...);
}

// The lowest value of a signed integer has no representable magnitude; as in the reference, that case is not treated.
template <typename T>
FK_HD_CNST auto abs(const T& x) {
    static_assert(std::is_fundamental_v<T>, "abs does not support non fundamental types");
    if constexpr (std::is_signed_v<T>) {
        return x < T(0) ? -x : x;
    } else {
        return x;
    }
}
} // namespace cxp
} // namespace fk
#endif
