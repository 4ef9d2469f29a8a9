// A string of fixed capacity that can be built, joined and compared in constant expressions: for names that are put
// together at compile time (kernel names, type descriptions).
//
// Interface of the reference's core/data/string.h:27-150: String<N> holds N - 1 characters and the terminator, deduces N
// from a literal, and offers size(), capacity(), operator[], at(), operator+ with strings and literals, substr(), c_str(),
// operator() (a std::string), ==, < and stream output.
#ifndef FK_CORE_STRING_H
#define FK_CORE_STRING_H

#include <cstddef>
#include <iostream>
#include <stdexcept>
#include <string>

namespace fk {
template <size_t N>
class String {
    static_assert(N >= 1, "a String holds at least its terminator");
    char chars[N] = {};

public:
    constexpr String() = default;
    constexpr String(const char (&literal)[N]) {
        for (size_t i = 0; i + 1 < N; ++i) chars[i] = literal[i];
        chars[N - 1] = '\0';
    }

    constexpr size_t size() const noexcept { return N - 1; }
    constexpr size_t capacity() const noexcept { return N; }
    constexpr char operator[](size_t index) const noexcept { return chars[index]; }
    constexpr char at(size_t index) const {
        if (index >= size()) throw std::out_of_range("String index out of range");
        return chars[index];
    }
    constexpr const char* c_str() const noexcept { return chars; }
    std::string operator()() const noexcept { return std::string(chars); }

    template <size_t M>
    constexpr String<N + M - 1> operator+(const String<M>& other) const noexcept {
        String<N + M - 1> joined{};
        for (size_t i = 0; i < size(); ++i) joined.set(i, chars[i]);
        for (size_t i = 0; i < other.size(); ++i) joined.set(size() + i, other[i]);
        return joined;
    }
    template <size_t M>
    constexpr String<N + M - 1> operator+(const char (&literal)[M]) const noexcept {
        return *this + String<M>(literal);
    }
    // `count` characters from `start` on (fewer when the string ends first), in a string of the same capacity
    constexpr String<N> substr(size_t start, size_t count) const {
        if (start > size()) throw std::out_of_range("String::substr start out of range");
        String<N> part{};
        for (size_t i = 0; i < count && start + i < size(); ++i) part.set(i, chars[start + i]);
        return part;
    }

    template <size_t M>
    constexpr bool operator==(const String<M>& other) const noexcept {
        if constexpr (N != M) {
            return false;
        } else {
            for (size_t i = 0; i < size(); ++i) {
                if (chars[i] != other[i]) return false;
            }
            return true;
        }
    }
    template <size_t M>
    constexpr bool operator==(const char (&literal)[M]) const noexcept {
        return *this == String<M>(literal);
    }
    template <size_t M>
    constexpr bool operator<(const String<M>& other) const noexcept {
        const size_t common = size() < other.size() ? size() : other.size();
        for (size_t i = 0; i < common; ++i) {
            if (chars[i] != other[i]) return chars[i] < other[i];
        }
        return size() < other.size();
    }

    constexpr void set(size_t index, char c) noexcept { chars[index] = c; } // building block of operator+ and substr
};
template <size_t N>
String(const char (&)[N]) -> String<N>;
} // namespace fk

template <size_t N>
inline std::ostream& operator<<(std::ostream& os, const fk::String<N>& str) {
    return os << str.c_str();
}
#endif
