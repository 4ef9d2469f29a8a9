// Math helpers that are usable in constant expressions and in device code alike.
//
// Follows the reference's core/constexpr_libs/constexpr_cmath.h:23-181: limits as variable templates, isnan/isinf
// without library calls, comparisons between integers of different signedness that never convert a negative value to
// unsigned, round half away from zero through an int cast, max/min over any number of equal-typed values (on a tie, or
// on an unordered comparison, the later argument wins), and abs.
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

template <typename T>
FK_HD_CNST bool isnan(T x) {
    return x != x;
}
template <typename T>
FK_HD_CNST bool isinf(T x) {
    return x == x && x != T(0) && x + x == x;
}

namespace detail {
template <typename T, typename U>
constexpr bool comparable_as_written = std::is_floating_point_v<T> || std::is_floating_point_v<U> || (std::is_signed_v<T> == std::is_signed_v<U>);
template <typename T, typename U>
constexpr void check_comparable() {
    static_assert(std::is_fundamental_v<T> && !std::is_same_v<T, bool>, "First parameter should be a fundamental type other than bool.");
    static_assert(std::is_fundamental_v<U> && !std::is_same_v<U, bool>, "Second parameter should be a fundamental type other than bool.");
}
} // namespace detail

template <typename T, typename U>
FK_HD_CNST bool cmp_equal(const T& t, const U& u) {
    detail::check_comparable<T, U>();
    if constexpr (detail::comparable_as_written<T, U>) {
        return t == u;
    } else if constexpr (std::is_signed_v<T>) {
        return t >= 0 && static_cast<std::make_unsigned_t<T>>(t) == u;
    } else {
        return u >= 0 && t == static_cast<std::make_unsigned_t<U>>(u);
    }
}
template <typename T, typename U>
FK_HD_CNST bool cmp_not_equal(const T& t, const U& u) {
    return !cmp_equal(t, u);
}
template <typename T, typename U>
FK_HD_CNST bool cmp_less(const T& t, const U& u) {
    detail::check_comparable<T, U>();
    if constexpr (detail::comparable_as_written<T, U>) {
        return t < u;
    } else if constexpr (std::is_signed_v<T>) {
        return t < 0 || static_cast<std::make_unsigned_t<T>>(t) < u;
    } else {
        return u >= 0 && t < static_cast<std::make_unsigned_t<U>>(u);
    }
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

// Half away from zero through an int cast; NaN and the infinities pass through.
template <typename T>
FK_HD_CNST T round(T x) {
    static_assert(std::is_floating_point_v<T>, "Input must be a floating-point type");
    if (isnan(x) || isinf(x)) return x;
    return (x > T(0)) ? static_cast<T>(static_cast<int>(x + T(0.5))) : static_cast<T>(static_cast<int>(x - T(0.5)));
}

template <typename T>
FK_HD_CNST T max(const T& value) {
    return value;
}
template <typename T, typename... Ts>
FK_HD_CNST T max(const T& first, const Ts&... rest) {
    static_assert((std::is_same_v<T, Ts> && ...), "All types must be the same");
    const T later = max(rest...);
    return first >= later ? first : later;
}
template <typename T>
FK_HD_CNST T min(const T& value) {
    return value;
}
template <typename T, typename... Ts>
FK_HD_CNST T min(const T& first, const Ts&... rest) {
    static_assert((std::is_same_v<T, Ts> && ...), "All types must be the same");
    const T later = min(rest...);
    return first <= later ? first : later;
}

// For the lowest value of a signed integer the result is not representable; as in the reference, that case is not treated.
template <typename T>
FK_HD_CNST auto abs(const T& x) {
    static_assert(std::is_fundamental_v<T>, "abs does not support non fundamental types");
    if constexpr (std::is_signed_v<T>) {
        return x < static_cast<T>(0) ? -x : x;
    } else {
        return x;
    }
}
} // namespace cxp
} // namespace fk
#endif
