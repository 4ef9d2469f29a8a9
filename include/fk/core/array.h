// A fixed-size array that is usable in constant expressions and device code, with the conveniences the vector types
// lack: run-time indexing, construction from a vector of the same base type, and a few helpers over array-like types.
//
// Follows the interface of the reference's core/data/array.h:24-254 (Array, ToArray, toArray, toVector, ArrayTraits,
// transformArray, getIndexArray, makeIndexArray, allValuesAre).  The storage here is a plain member array: the reference
// overlays named members x, y, z, w on it through a union, which cannot be read back in a constant expression.
#ifndef FK_CORE_ARRAY_H
#define FK_CORE_ARRAY_H

#include <array>

#include "fk/core/type_utils.h"
#include "fk/core/vector_types.h"

namespace fk {
namespace detail {
template <typename T, size_t SIZE, bool VECTOR = (SIZE >= 1 && SIZE <= 4 && std::is_fundamental_v<T>)>
struct ArrayVector {
    struct None {}; // no vector type has this shape
    using type = None;
};
template <typename T, size_t SIZE>
struct ArrayVector<T, SIZE, true> {
    using type = typename VectorType<T, static_cast<int>(SIZE)>::type_v;
};
} // namespace detail

template <typename T, size_t SIZE>
struct Array {
    enum { size = SIZE };
    using Vector = typename detail::ArrayVector<T, SIZE>::type;
    T at[SIZE == 0 ? 1 : SIZE];

    constexpr Array() = default;
    // every element set to one value
    __host__ __device__ constexpr Array(const T& initValue) : at{} {
        for (size_t i = 0; i < SIZE; ++i) at[i] = initValue;
    }
    // one value per element
    template <typename... Types, std::enable_if_t<(sizeof...(Types) == SIZE && SIZE > 1), int> = 0>
    __host__ __device__ constexpr Array(const Types&... values) : at{ static_cast<T>(values)... } {
        static_assert((std::is_same_v<T, Types> && ...), "Not all input types are the expected type T");
    }
    // the channels of a vector
    __host__ __device__ constexpr Array(const Vector& other) : at{} { fromVector(other, std::make_integer_sequence<int, static_cast<int>(SIZE)>{}); }
    __host__ __device__ constexpr Array& operator=(const Vector& other) {
        fromVector(other, std::make_integer_sequence<int, static_cast<int>(SIZE)>{});
        return *this;
    }
    __host__ __device__ constexpr T operator[](const size_t& index) const { return at[index]; }
    // Same element through a chain of selects instead of an address computation, which lets the compiler keep a
    // private Array in registers.
    __host__ __device__ constexpr T operator()(const int& index) const {
        T value = at[0];
        for (size_t i = 1; i < SIZE; ++i) value = (static_cast<int>(i) == index) ? at[i] : value;
        return value;
    }

private:
    template <int... K>
    __host__ __device__ constexpr void fromVector(const Vector& other, std::integer_sequence<int, K...>) {
        if constexpr (validCUDAVec<Vector>) ((at[K] = vget<K>(other)), ...);
    }
};

template <typename CUDAVector>
using ToArray = Array<VBase<CUDAVector>, static_cast<size_t>(cn<CUDAVector>)>;
template <typename V>
FK_HD_CNST ToArray<V> toArray(const V& vector) {
    return ToArray<V>(vector); // a scalar gives an array of one element
}
namespace detail {
template <typename T, size_t SIZE, size_t... Idx>
FK_HD_CNST VectorType_t<T, static_cast<int>(SIZE)> to_vector(const Array<T, SIZE>& a, std::index_sequence<Idx...>) {
    return VectorType_t<T, static_cast<int>(SIZE)>{ a.at[Idx]... };
}
} // namespace detail
template <typename T, size_t SIZE>
FK_HD_CNST VectorType_t<T, static_cast<int>(SIZE)> toVector(const Array<T, SIZE>& a) {
    static_assert(SIZE >= 1 && SIZE <= 4, "No Vector types available with size greater than 4");
    if constexpr (SIZE == 1) {
        return a.at[0];
    } else {
        return detail::to_vector(a, std::make_index_sequence<SIZE>{});
    }
}

// element type and size of fk::Array, std::array and anything else shaped like template <typename, size_t>
template <typename ArrayLike>
struct ArrayTraits;
template <template <typename, size_t> class ArrayLike, typename T, size_t N>
struct ArrayTraits<ArrayLike<T, N>> {
    using type = T;
    static constexpr size_t size = N;
};
template <typename ArrayLike>
constexpr size_t arraySize = ArrayTraits<ArrayLike>::size;
template <typename ArrayLike>
using ArrayType = typename ArrayTraits<ArrayLike>::type;
template <size_t BATCH, typename... ArrayTypes>
constexpr bool allArraysSameSize_v = and_v<(arraySize<ArrayTypes> == BATCH)...>;

namespace detail {
template <template <typename, size_t> class ArrayLike, typename T, size_t N, typename F, size_t... Is>
inline constexpr auto transform_array(const ArrayLike<T, N>& input, F&& func, std::index_sequence<Is...>) {
    using Result = decltype(func(std::declval<std::decay_t<decltype(input[0])>>()));
    return ArrayLike<Result, N>{ { func(input[Is])... } };
}
template <typename ArrayT, size_t... Idx>
FK_HD_CNST ArrayT index_array(std::index_sequence<Idx...>) {
    return ArrayT{ Idx... };
}
template <typename T, typename ArrayT, size_t... Idx>
FK_HD_CNST bool all_values_are(const T& value, const ArrayT& values, std::index_sequence<Idx...>) {
    return ((values[Idx] == value) && ...);
}
} // namespace detail
// func applied to every element, in an array of the same kind
template <typename ArrayLike, typename F>
inline constexpr auto transformArray(const ArrayLike& input, F&& func) {
    return detail::transform_array(input, std::forward<F>(func), std::make_index_sequence<arraySize<ArrayLike>>{});
}
// { 0, 1, ..., N-1 }
template <template <typename, size_t> class ArrayLike, typename T, size_t N>
FK_HD_CNST ArrayLike<size_t, N> getIndexArray(const ArrayLike<T, N>&) {
    return detail::index_array<ArrayLike<size_t, N>>(std::make_index_sequence<N>{});
}
template <size_t N>
FK_HD_CNST Array<size_t, N> makeIndexArray() {
    return detail::index_array<Array<size_t, N>>(std::make_index_sequence<N>{});
}
template <template <typename, size_t> class ArrayLike, typename T, size_t N>
FK_HD_CNST bool allValuesAre(const T& value, const ArrayLike<T, N>& values) {
    return detail::all_values_are(value, values, std::make_index_sequence<N>{});
}
} // namespace fk
#endif
