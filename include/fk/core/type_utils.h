// Compile-time helpers that user code of the library builds on: boolean folds, TypeList queries and edits, filtered
// index sequences, a plain aggregate Tuple and std::array fillers.
//
// Same names and results as the reference's core/utils/template_operations.h (and_v, or_v), core/utils/type_lists.h
// (TypeAt_t, TypeListCat_t, InsertTypeFront_t / InsertTypeBack_t / InsertType_t, one_of_v, TypeIndex_v,
// EquivalentType_t, isTypeList), core/utils/parameter_pack_utils.h (filtered_integer_sequence_t,
// filtered_index_sequence_t, get_index, get_integer, NotUnaryRestriction), core/data/tuple.h (Tuple, TupleUtil, get, cat,
// tuple_insert) and core/data/array.h (make_set_std_array), as their tests/data/test_typelist.h, test_tuple.h and
// tests/operation/test_filtered_index_sequence.h use them.
#ifndef FK_CORE_TYPE_UTILS_H
#define FK_CORE_TYPE_UTILS_H

#include <array>
#include <type_traits>
#include <utility>

#include "fk/core/utils.h"

namespace fk {

template <bool... Values>
constexpr bool and_v = (Values && ...);
template <bool... Values>
constexpr bool or_v = (Values || ...);

// ---- TypeList --------------------------------------------------------------------------------------------------
template <typename T>
constexpr bool isTypeList = false;
template <typename... Ts>
constexpr bool isTypeList<TypeList<Ts...>> = true;

namespace detail {
template <size_t N, typename List>
struct TypeAtImpl;
template <size_t N, typename First, typename... Rest>
struct TypeAtImpl<N, TypeList<First, Rest...>> : TypeAtImpl<N - 1, TypeList<Rest...>> {};
template <typename First, typename... Rest>
struct TypeAtImpl<0, TypeList<First, Rest...>> {
    using type = First;
};
template <typename... Lists>
struct TypeListCatImpl;
template <typename... As>
struct TypeListCatImpl<TypeList<As...>> {
    using type = TypeList<As...>;
};
template <typename... As, typename... Bs, typename... More>
struct TypeListCatImpl<TypeList<As...>, TypeList<Bs...>, More...> : TypeListCatImpl<TypeList<As..., Bs...>, More...> {};
// the first N types of a list, and the rest
template <size_t N, typename Taken, typename Left, bool DONE = (N == 0)>
struct SplitAt;
template <size_t N, typename... Taken, typename... Left>
struct SplitAt<N, TypeList<Taken...>, TypeList<Left...>, true> {
    using head = TypeList<Taken...>;
    using tail = TypeList<Left...>;
};
template <size_t N, typename... Taken, typename Next, typename... Left>
struct SplitAt<N, TypeList<Taken...>, TypeList<Next, Left...>, false> : SplitAt<N - 1, TypeList<Taken..., Next>, TypeList<Left...>> {};
template <typename T, typename List>
struct IndexOf;
template <typename T, typename... Rest>
struct IndexOf<T, TypeList<T, Rest...>> : std::integral_constant<size_t, 0> {};
template <typename T, typename First, typename... Rest>
struct IndexOf<T, TypeList<First, Rest...>> : std::integral_constant<size_t, 1 + IndexOf<T, TypeList<Rest...>>::value> {};
} // namespace detail

// element N of a list; -1 names the last one
template <int N, typename List>
using TypeAt_t = typename detail::TypeAtImpl<(N < 0 ? static_cast<size_t>(List::size) - 1 : static_cast<size_t>(N)), List>::type;
template <typename... Lists>
using TypeListCat_t = typename detail::TypeListCatImpl<Lists...>::type;
template <typename List, typename T>
using InsertTypeBack_t = TypeListCat_t<List, TypeList<T>>;
template <typename T, typename List>
using InsertTypeFront_t = TypeListCat_t<TypeList<T>, List>;
// T becomes element N; the elements from N on move one place back
template <size_t N, typename T, typename List>
using InsertType_t = TypeListCat_t<typename detail::SplitAt<N, TypeList<>, List>::head, TypeList<T>, typename detail::SplitAt<N, TypeList<>, List>::tail>;

template <typename T, typename List>
constexpr bool one_of_v = false;
template <typename T, typename... Ts>
constexpr bool one_of_v<T, TypeList<Ts...>> = (std::is_same_v<T, Ts> || ...);
template <typename T, typename List>
constexpr size_t TypeIndex_v = detail::IndexOf<T, List>::value;
// the type of ListTwo at the place T has in ListOne
template <typename T, typename ListOne, typename ListTwo>
using EquivalentType_t = TypeAt_t<static_cast<int>(TypeIndex_v<T, ListOne>), ListTwo>;
// the list without element N
template <size_t N, typename List>
using RemoveType_t = TypeListCat_t<typename detail::SplitAt<N, TypeList<>, List>::head,
                                   typename detail::SplitAt<1, TypeList<>, typename detail::SplitAt<N, TypeList<>, List>::tail>::tail>;
template <typename T, typename List>
constexpr bool all_of_v = false;
template <typename T, typename... Ts>
constexpr bool all_of_v<T, TypeList<Ts...>> = (std::is_same_v<T, Ts> && ...);
// the same queries as class templates
template <typename T>
struct IsTypeList : std::bool_constant<isTypeList<T>> {};
template <typename T, typename List>
struct one_of : std::bool_constant<one_of_v<T, List>> {};
template <typename T, typename List>
struct all_of : std::bool_constant<all_of_v<T, List>> {};
template <typename T, typename List>
struct TypeIndex : std::integral_constant<size_t, TypeIndex_v<T, List>> {};
template <typename ListOne, typename ListTwo>
struct TypeListCat {
    using type = TypeListCat_t<ListOne, ListTwo>;
};
// an enumerator as a type
template <typename Enum, Enum VALUE>
struct EnumType {};
template <typename Enum, Enum VALUE>
using E_t = EnumType<Enum, VALUE>;

template <typename... Types>
using FirstType_t = TypeAt_t<0, TypeList<Types...>>;
template <typename... Types>
using LastType_t = TypeAt_t<-1, TypeList<Types...>>;
template <typename... IOps>
using FirstInstantiableOperationInputType_t = typename FirstType_t<IOps...>::Operation::InputType;
template <typename... IOps>
using LastInstantiableOperationOutputType_t = typename LastType_t<IOps...>::Operation::OutputType;

// ---- integer sequences and parameter packs -------------------------------------------------------------------------
// Position of a value in an integer sequence (-1 when absent), and membership.
template <typename T, T ELEMENT>
struct Find {
    template <T... Sequence>
    FK_HD_STATIC int in(std::integer_sequence<T, Sequence...>) {
        int position = -1, i = 0;
        ((position = (position < 0 && Sequence == ELEMENT) ? i : position, ++i), ...);
        return position;
    }
    template <T... Sequence>
    FK_HD_STATIC bool one_of(std::integer_sequence<T, Sequence...>) {
        return ((Sequence == ELEMENT) || ...);
    }
};
template <typename T, T START, T... Ints>
FK_HD_CNST auto make_integer_sequence_from(const std::integer_sequence<T, Ints...>&) {
    return std::integer_sequence<T, (START + Ints)...>{};
}
template <size_t N>
constexpr auto indexSequence = std::make_index_sequence<N>{};
// argument INDEX of a call
template <int INDEX, typename T, typename... Args>
FK_HD_CNST const auto& get(const T& current, const Args&... args) {
    static_assert(INDEX >= 0 && static_cast<int>(sizeof...(Args)) + 1 > INDEX, "Index out of range when looking for a parameter in a parameter pack.");
    if constexpr (INDEX == 0) {
        return current;
    } else {
        return get<INDEX - 1>(args...);
    }
}
template <typename... Args>
FK_HD_CNST const auto& ppFirst(const Args&... args) {
    return get<0>(args...);
}
template <typename... Args>
FK_HD_CNST const auto& ppLast(const Args&... args) {
    return get<static_cast<int>(sizeof...(Args)) - 1>(args...);
}

// ---- filtered sequences ------------------------------------------------------------------------------------------
// The positions of the types of a list that comply with a restriction (`Restriction::template complies<T>()`), in order.
namespace detail {
template <typename Int, Int CURRENT, typename Restriction, typename List, typename Sequence>
struct FilteredSequence;
template <typename Int, Int CURRENT, typename Restriction, Int... Found>
struct FilteredSequence<Int, CURRENT, Restriction, TypeList<>, std::integer_sequence<Int, Found...>> {
    using type = std::integer_sequence<Int, Found...>;
};
template <typename Int, Int CURRENT, typename Restriction, typename First, typename... Rest, Int... Found>
struct FilteredSequence<Int, CURRENT, Restriction, TypeList<First, Rest...>, std::integer_sequence<Int, Found...>>
    : FilteredSequence<Int, CURRENT + 1, Restriction, TypeList<Rest...>,
                       std::conditional_t<Restriction::template complies<First>(), std::integer_sequence<Int, Found..., CURRENT>, std::integer_sequence<Int, Found...>>> {};
template <typename Int, size_t N, typename Sequence>
struct SequenceAt;
template <typename Int, size_t N, Int First, Int... Rest>
struct SequenceAt<Int, N, std::integer_sequence<Int, First, Rest...>> : SequenceAt<Int, N - 1, std::integer_sequence<Int, Rest...>> {};
template <typename Int, Int First, Int... Rest>
struct SequenceAt<Int, 0, std::integer_sequence<Int, First, Rest...>> : std::integral_constant<Int, First> {};
} // namespace detail

template <typename Int, typename Restriction, typename List>
using filtered_integer_sequence_t = typename detail::FilteredSequence<Int, Int(0), Restriction, List, std::integer_sequence<Int>>::type;
template <typename Restriction, typename List>
using filtered_index_sequence_t = filtered_integer_sequence_t<size_t, Restriction, List>;
template <typename Int, size_t N, typename Sequence>
constexpr Int get_integer = detail::SequenceAt<Int, N, Sequence>::value;
template <size_t N, typename Sequence>
constexpr size_t get_index = get_integer<size_t, N, Sequence>;
template <size_t N, size_t... Idx>
constexpr size_t get_index_f(const std::index_sequence<Idx...>&) {
    return get_index<N, std::index_sequence<Idx...>>;
}

// ---- Tuple -------------------------------------------------------------------------------------------------------
// An aggregate: Tuple<int, float3> t{ 1, { 2.f, 3.f, 4.f } } works in constant expressions and in device code.
template <typename... Types>
struct Tuple {};
template <typename T>
struct Tuple<T> {
    T instance;
    enum { size = 1 };
};
template <typename T, typename... Rest>
struct Tuple<T, Rest...> {
    T instance;
    Tuple<Rest...> next;
    enum { size = sizeof...(Rest) + 1 };
};

namespace detail {
template <int INDEX, typename List>
struct TupleElement; // shared with OperationTuple (fk/core/operation_model.h)
template <int INDEX, typename First, typename... Rest>
struct TupleElement<INDEX, Tuple<First, Rest...>> : TupleElement<INDEX - 1, Tuple<Rest...>> {};
template <typename First, typename... Rest>
struct TupleElement<0, Tuple<First, Rest...>> {
    using type = First;
};
} // namespace detail

struct TupleUtil {
    template <int INDEX, typename... Types>
    FK_HD_STATIC auto& get(Tuple<Types...>& t) {
        static_assert(INDEX >= 0 && INDEX < static_cast<int>(sizeof...(Types)), "Index out of range.");
        if constexpr (INDEX == 0) return t.instance;
        else return get<INDEX - 1>(t.next);
    }
    template <int INDEX, typename... Types>
    FK_HD_STATIC const auto& get(const Tuple<Types...>& t) {
        static_assert(INDEX >= 0 && INDEX < static_cast<int>(sizeof...(Types)), "Index out of range.");
        if constexpr (INDEX == 0) return t.instance;
        else return get<INDEX - 1>(t.next);
    }
    template <typename... As, typename... Bs>
    FK_HD_STATIC Tuple<As..., Bs...> cat(const Tuple<As...>& a, const Tuple<Bs...>& b) {
        return cat_impl(a, b, std::make_integer_sequence<int, static_cast<int>(sizeof...(As))>{}, std::make_integer_sequence<int, static_cast<int>(sizeof...(Bs))>{});
    }
    // `value` becomes element INDEX; the elements from INDEX on move one place back
    template <int INDEX, typename T, typename... Types>
    FK_HD_STATIC auto tuple_insert(const T& value, const Tuple<Types...>& t) {
        static_assert(INDEX >= 0 && INDEX <= static_cast<int>(sizeof...(Types)), "Index out of range.");
        return insert_impl<T>(value, t, std::make_integer_sequence<int, INDEX>{}, std::make_integer_sequence<int, static_cast<int>(sizeof...(Types)) - INDEX>{});
    }

private:
    template <typename... As, typename... Bs, int... Ia, int... Ib>
    FK_HD_STATIC Tuple<As..., Bs...> cat_impl(const Tuple<As...>& a, const Tuple<Bs...>& b, std::integer_sequence<int, Ia...>, std::integer_sequence<int, Ib...>) {
        return Tuple<As..., Bs...>{ get<Ia>(a)..., get<Ib>(b)... };
    }
    template <typename T, typename... Types, int... Before, int... After>
    FK_HD_STATIC auto insert_impl(const T& value, const Tuple<Types...>& t, std::integer_sequence<int, Before...>, std::integer_sequence<int, After...>) {
        using Source = Tuple<Types...>;
        return Tuple<typename detail::TupleElement<Before, Source>::type..., T,
                     typename detail::TupleElement<static_cast<int>(sizeof...(Before)) + After, Source>::type...>{
            get<Before>(t)..., value, get<static_cast<int>(sizeof...(Before)) + After>(t)...
        };
    }
};

template <int INDEX, typename... Types>
FK_HD_CNST auto& get(Tuple<Types...>& t) { return TupleUtil::get<INDEX>(t); }
template <int INDEX, typename... Types>
FK_HD_CNST const auto& get(const Tuple<Types...>& t) { return TupleUtil::get<INDEX>(t); }
template <typename... As, typename... Bs>
FK_HD_CNST Tuple<As..., Bs...> cat(const Tuple<As...>& a, const Tuple<Bs...>& b) { return TupleUtil::cat(a, b); }
template <int INDEX, typename T, typename... Types>
FK_HD_CNST auto tuple_insert(const T& value, const Tuple<Types...>& t) { return TupleUtil::tuple_insert<INDEX, T>(value, t); }
template <typename... Types>
FK_HD_CNST Tuple<std::decay_t<Types>...> make_tuple(const Types&... values) { return Tuple<std::decay_t<Types>...>{ values... }; }

template <typename T, typename TupleLike>
FK_HD_CNST auto tuple_insert_back(const TupleLike& t, const T& value) { return TupleUtil::tuple_insert<static_cast<int>(TupleLike::size), T>(value, t); }

template <typename T>
struct isTuple : std::false_type {};
template <typename... Types>
struct isTuple<Tuple<Types...>> : std::true_type {};
template <typename T>
constexpr bool isTuple_v = isTuple<std::decay_t<T>>::value;

namespace detail {
template <typename TupleType>
struct TupleTypes;
template <typename... Types>
struct TupleTypes<Tuple<Types...>> {
    using type = TypeList<Types...>;
};
} // namespace detail
template <typename TupleType>
using ToTypeList = typename detail::TupleTypes<TupleType>::type;
template <int INDEX, typename TupleType>
using get_t = TypeAt_t<INDEX, ToTypeList<TupleType>>;

// f(get<0>(t), get<1>(t), ...)
namespace detail {
template <typename F, typename TupleType, size_t... Idx>
FK_HD_CNST decltype(auto) apply_to_elements(F&& f, TupleType& t, std::index_sequence<Idx...>) {
    return std::forward<F>(f)(get<static_cast<int>(Idx)>(t)...);
}
} // namespace detail
template <typename F, typename TupleType>
FK_HD_CNST decltype(auto) apply(F&& f, TupleType& t) {
    return detail::apply_to_elements(std::forward<F>(f), t, std::make_index_sequence<static_cast<size_t>(TupleType::size)>{});
}

// ---- arrays ------------------------------------------------------------------------------------------------------
namespace detail {
template <typename T, size_t... Idx>
FK_HD_CNST std::array<T, sizeof...(Idx)> fill_array(const T& value, std::index_sequence<Idx...>) {
    return { { (static_cast<void>(Idx), value)... } };
}
} // namespace detail
template <size_t BATCH, typename T>
FK_HD_CNST std::array<T, BATCH> make_set_std_array(const T& value) {
    return detail::fill_array(value, std::make_index_sequence<BATCH>{});
}

} // namespace fk
#endif
