// Plain vector structs (uchar3, float4, ...) with the byte layout image buffers are stored in, their traits, and
// element-wise operators with the usual arithmetic conversions per channel.
//
// Layouts follow the reference's core/data/vector_types.h:23-313 (1- and 3-channel types keep the base alignment,
// 2-/4-channel types align to their size up to 16 bytes); traits and operators follow
// core/utils/cuda_vector_utils.h:26-602 (VectorType_t, cn, VBase, make_, make_set, operator result =
// vector of decltype(base op base)).  The structs are this library's own: no runtime header defines them.
#ifndef FK_CORE_VECTOR_TYPES_H
#define FK_CORE_VECTOR_TYPES_H

#include "fk/core/utils.h"

namespace fk {

#define FK_DEFINE_VECTOR_FAMILY(NAME, BASE, A2, A4)                                                                    \
    struct NAME##1 { BASE x; };                                                                                        \
    struct alignas(A2) NAME##2 { BASE x, y; };                                                                         \
    struct NAME##3 { BASE x, y, z; };                                                                                  \
    struct alignas(A4) NAME##4 { BASE x, y, z, w; };

// Vectors of bool (the result of comparing two vectors) also convert to one bool: true when every channel is.
struct bool1 { bool x; __host__ __device__ constexpr operator bool() const { return x; } };
struct bool2 { bool x, y; __host__ __device__ constexpr operator bool() const { return x && y; } };
struct bool3 { bool x, y, z; __host__ __device__ constexpr operator bool() const { return x && y && z; } };
struct bool4 { bool x, y, z, w; __host__ __device__ constexpr operator bool() const { return x && y && z && w; } };
using Bool1 = bool1;
using Bool2 = bool2;
using Bool3 = bool3;
using Bool4 = bool4;
// All / any channel of a bool vector.
struct Bool {
    static constexpr __host__ __device__ bool vAnd(const bool1& v) { return v.x; }
    static constexpr __host__ __device__ bool vAnd(const bool2& v) { return v.x && v.y; }
    static constexpr __host__ __device__ bool vAnd(const bool3& v) { return v.x && v.y && v.z; }
    static constexpr __host__ __device__ bool vAnd(const bool4& v) { return v.x && v.y && v.z && v.w; }
    static constexpr __host__ __device__ bool vOr(const bool1& v) { return v.x; }
    static constexpr __host__ __device__ bool vOr(const bool2& v) { return v.x || v.y; }
    static constexpr __host__ __device__ bool vOr(const bool3& v) { return v.x || v.y || v.z; }
    static constexpr __host__ __device__ bool vOr(const bool4& v) { return v.x || v.y || v.z || v.w; }
};
FK_DEFINE_VECTOR_FAMILY(char, signed char, 2, 4)
FK_DEFINE_VECTOR_FAMILY(uchar, unsigned char, 2, 4)
FK_DEFINE_VECTOR_FAMILY(short, short, 4, 8)
FK_DEFINE_VECTOR_FAMILY(ushort, unsigned short, 4, 8)
FK_DEFINE_VECTOR_FAMILY(int, int, 8, 16)
FK_DEFINE_VECTOR_FAMILY(uint, unsigned int, 8, 16)
FK_DEFINE_VECTOR_FAMILY(long, long, 16, 16)
FK_DEFINE_VECTOR_FAMILY(ulong, unsigned long, 16, 16)
FK_DEFINE_VECTOR_FAMILY(longlong, long long, 16, 16)
FK_DEFINE_VECTOR_FAMILY(ulonglong, unsigned long long, 16, 16)
FK_DEFINE_VECTOR_FAMILY(float, float, 8, 16)
FK_DEFINE_VECTOR_FAMILY(double, double, 16, 16)
#undef FK_DEFINE_VECTOR_FAMILY

static_assert(sizeof(uchar3) == 3 && alignof(uchar3) == 1, "uchar3 must be 3 packed bytes");
static_assert(sizeof(uchar4) == 4 && alignof(uchar4) == 4, "uchar4 must be one dword");
static_assert(sizeof(float3) == 12 && alignof(float3) == 4, "float3 must be 12 packed bytes");
static_assert(sizeof(float4) == 16 && alignof(float4) == 16, "float4 must be 16 aligned bytes");

// ---- traits ----------------------------------------------------------------------------------------------------
template <typename T>
struct VectorTraits {
    using base = T;
    static constexpr int channels = 1;
    static constexpr bool is_vector = false;
    enum { bytes = sizeof(T) };
};

template <typename Base, int N>
struct VectorType;

#define FK_VECTOR_TRAITS(NAME, BASE)                                                                                   \
    template <> struct VectorTraits<NAME##1> { using base = BASE; static constexpr int channels = 1; static constexpr bool is_vector = true; enum { bytes = sizeof(BASE) }; }; \
    template <> struct VectorTraits<NAME##2> { using base = BASE; static constexpr int channels = 2; static constexpr bool is_vector = true; enum { bytes = sizeof(BASE) }; }; \
    template <> struct VectorTraits<NAME##3> { using base = BASE; static constexpr int channels = 3; static constexpr bool is_vector = true; enum { bytes = sizeof(BASE) }; }; \
    template <> struct VectorTraits<NAME##4> { using base = BASE; static constexpr int channels = 4; static constexpr bool is_vector = true; enum { bytes = sizeof(BASE) }; }; \
    template <> struct VectorType<BASE, 1> { using type = BASE; using type_v = NAME##1; };                             \
    template <> struct VectorType<BASE, 2> { using type = NAME##2; using type_v = NAME##2; };                          \
    template <> struct VectorType<BASE, 3> { using type = NAME##3; using type_v = NAME##3; };                          \
    template <> struct VectorType<BASE, 4> { using type = NAME##4; using type_v = NAME##4; };

FK_VECTOR_TRAITS(bool, bool)
FK_VECTOR_TRAITS(char, signed char)
FK_VECTOR_TRAITS(uchar, unsigned char)
FK_VECTOR_TRAITS(short, short)
FK_VECTOR_TRAITS(ushort, unsigned short)
FK_VECTOR_TRAITS(int, int)
FK_VECTOR_TRAITS(uint, unsigned int)
FK_VECTOR_TRAITS(long, long)
FK_VECTOR_TRAITS(ulong, unsigned long)
FK_VECTOR_TRAITS(longlong, long long)
FK_VECTOR_TRAITS(ulonglong, unsigned long long)
FK_VECTOR_TRAITS(float, float)
FK_VECTOR_TRAITS(double, double)
#undef FK_VECTOR_TRAITS

// plain `char` maps onto the family of its signedness
template <>
struct VectorTraits<char> {
    using base = std::conditional_t<std::is_unsigned_v<char>, unsigned char, signed char>;
    static constexpr int channels = 1;
    static constexpr bool is_vector = false;
    enum { bytes = 1 };
};
template <int N>
struct VectorType<char, N> : VectorType<std::conditional_t<std::is_unsigned_v<char>, unsigned char, signed char>, N> {};

template <typename Base, int N>
using VectorType_t = typename VectorType<Base, N>::type;

template <typename T>
constexpr bool validCUDAVec = VectorTraits<std::remove_cv_t<T>>::is_vector;

// Number of channels; 1 for scalars.  cv-qualified vector types count as scalars here, as they do in the reference
// (core/utils/cuda_vector_utils.h:99-113 matches unqualified types only).
template <typename T>
constexpr int cn = VectorTraits<T>::channels;

template <typename T>
using VBase = typename VectorTraits<std::remove_cv_t<T>>::base;

// ---- lists of the types above, and what may be combined with what (core/utils/cuda_vector_utils.h:74-97,308-367) -----
template <uint CHANNELS>
using VectorTypeList = TypeList<VectorType_t<bool, CHANNELS>, VectorType_t<uchar, CHANNELS>, VectorType_t<schar, CHANNELS>,
                                VectorType_t<ushort, CHANNELS>, VectorType_t<short, CHANNELS>, VectorType_t<uint, CHANNELS>,
                                VectorType_t<int, CHANNELS>, VectorType_t<ulong, CHANNELS>, VectorType_t<long, CHANNELS>,
                                VectorType_t<ulonglong, CHANNELS>, VectorType_t<longlong, CHANNELS>, VectorType_t<float, CHANNELS>,
                                VectorType_t<double, CHANNELS>>;
using FloatingTypes = TypeList<float, double>;
using IntegralTypes = TypeList<uchar, char, schar, ushort, short, uint, int, ulong, long, ulonglong, longlong>;
using IntegralBaseTypes = TypeList<uchar, schar, ushort, short, uint, int, ulong, long, ulonglong, longlong>;
using StandardTypes = TypeList<bool, uchar, char, schar, ushort, short, uint, int, ulong, long, ulonglong, longlong, float, double>;
using BaseTypes = TypeList<bool, uchar, schar, ushort, short, uint, int, ulong, long, ulonglong, longlong, float, double>;
using VOne = TypeList<bool1, uchar1, char1, ushort1, short1, uint1, int1, ulong1, long1, ulonglong1, longlong1, float1, double1>;
using VTwo = VectorTypeList<2>;
using VThree = VectorTypeList<3>;
using VFour = VectorTypeList<4>;
using VAll = typename TypeList<VOne, VTwo, VThree, VFour>::type;

template <typename T>
struct IsCudaVector : std::bool_constant<validCUDAVec<T>> {};
template <typename I1, typename I2>
struct BothIntegrals : std::bool_constant<std::is_integral_v<VBase<I1>> && std::is_integral_v<VBase<I2>>> {};
template <typename I1, typename I2>
struct AreVVEqCN : std::bool_constant<validCUDAVec<I1> && validCUDAVec<I2> && cn<I1> == cn<I2>> {};
template <typename I1, typename I2>
struct AreSV : std::bool_constant<std::is_fundamental_v<I1> && validCUDAVec<I2>> {};
template <typename I1, typename I2>
struct AreVS : std::bool_constant<validCUDAVec<I1> && std::is_fundamental_v<I2>> {};
template <typename T>
struct CanUnary : std::bool_constant<validCUDAVec<T>> {};
template <typename I1, typename I2>
struct CanBinary : std::bool_constant<AreVVEqCN<I1, I2>::value || AreSV<I1, I2>::value || AreVS<I1, I2>::value> {};
template <typename I1, typename I2>
struct CanBinaryBitwise : std::bool_constant<CanBinary<I1, I2>::value && BothIntegrals<I1, I2>::value> {};
template <typename I1, typename I2>
struct CanCompound : std::bool_constant<AreVVEqCN<I1, I2>::value || AreVS<I1, I2>::value> {};
template <typename I1, typename I2>
struct CanCompoundLogical : std::bool_constant<CanCompound<I1, I2>::value && BothIntegrals<I1, I2>::value> {};

// ---- channel access and construction ------------------------------------------------------------------------------
template <int I, typename T>
FK_HD_CNST auto vget(const T& v) {
    if constexpr (!validCUDAVec<T>) {
        return v;
    } else if constexpr (I == 0) {
        return v.x;
    } else if constexpr (I == 1) {
        return v.y;
    } else if constexpr (I == 2) {
        return v.z;
    } else {
        return v.w;
    }
}

template <typename T>
FK_HD_CNST VBase<T> vectorAt(int idx, const T& v) {
    if constexpr (!validCUDAVec<T>) {
        return v;
    } else {
        if (idx == 0) return v.x;
        if constexpr (cn<T> >= 2) { if (idx == 1) return v.y; }
        if constexpr (cn<T> >= 3) { if (idx == 2) return v.z; }
        if constexpr (cn<T> >= 4) { if (idx == 3) return v.w; }
        return v.x;
    }
}

// The reference's spellings of the two accessors above (core/utils/cuda_vector_utils.h:160-229).
template <int IDX, typename T>
FK_HD_CNST auto VectorAt(const T& v) {
    static_assert(IDX >= 0 && IDX < cn<T>, "Index out of range for this vector type");
    return vget<IDX>(v);
}
template <typename T>
FK_HD_CNST VBase<T> VectorAt(const int& idx, const T& v) {
    return vectorAt(idx, v);
}

// make_<T>(a, b, ...): every argument is cast to T's base type (core/utils/cuda_vector_utils.h:235-265)
template <typename T, typename... Numbers>
FK_HD_CNST T make_(const Numbers&... pack) {
    if constexpr (validCUDAVec<T>) {
        static_assert(sizeof...(Numbers) <= cn<T>, "make_: at most one argument per channel (channels left out are zero)");
        return T{ static_cast<VBase<T>>(pack)... };
    } else {
        static_assert(sizeof...(Numbers) == 1, "make_: a scalar takes one argument");
        return (static_cast<T>(pack), ...);
    }
}

// make_set<T>(v): all channels set to v
template <typename T, typename V>
FK_HD_CNST T make_set(const V& v) {
    if constexpr (!validCUDAVec<T>) {
        return static_cast<T>(v);
    } else if constexpr (cn<T> == 1) {
        return make_<T>(v);
    } else if constexpr (cn<T> == 2) {
        return make_<T>(v, v);
    } else if constexpr (cn<T> == 3) {
        return make_<T>(v, v, v);
    } else {
        return make_<T>(v, v, v, v);
    }
}

namespace detail {
// Applies F channel by channel to (a, b); scalars broadcast.  The result vector has the base type that the
// scalar expression yields, so uchar*uchar gives int channels and uchar*float gives float channels.
template <typename F, typename A, typename B>
FK_HD_CNST auto vec_binary(const A& a, const B& b) {
    constexpr int N = cn<A> > cn<B> ? cn<A> : cn<B>;
    static_assert(!validCUDAVec<A> || !validCUDAVec<B> || cn<A> == cn<B>, "Vectors must have the same number of channels");
    using R = decltype(F::apply(vget<0>(a), vget<0>(b)));
    using O = typename VectorType<R, N>::type_v;
    if constexpr (N == 1) {
        return O{ F::apply(vget<0>(a), vget<0>(b)) };
    } else if constexpr (N == 2) {
        return O{ F::apply(vget<0>(a), vget<0>(b)), F::apply(vget<1>(a), vget<1>(b)) };
    } else if constexpr (N == 3) {
        return O{ F::apply(vget<0>(a), vget<0>(b)), F::apply(vget<1>(a), vget<1>(b)), F::apply(vget<2>(a), vget<2>(b)) };
    } else {
        return O{ F::apply(vget<0>(a), vget<0>(b)), F::apply(vget<1>(a), vget<1>(b)), F::apply(vget<2>(a), vget<2>(b)),
                  F::apply(vget<3>(a), vget<3>(b)) };
    }
}
#define FK_BINARY_FUNCTOR(NAME, OP)                                                                                    \
    struct NAME {                                                                                                      \
        template <typename X, typename Y>                                                                              \
        FK_HD_STATIC auto apply(const X& x, const Y& y) { return x OP y; }                                             \
    };
FK_BINARY_FUNCTOR(FnAdd, +)
FK_BINARY_FUNCTOR(FnSub, -)
FK_BINARY_FUNCTOR(FnMul, *)
FK_BINARY_FUNCTOR(FnDiv, /)
FK_BINARY_FUNCTOR(FnEq, ==)
FK_BINARY_FUNCTOR(FnNe, !=)
FK_BINARY_FUNCTOR(FnGt, >)
FK_BINARY_FUNCTOR(FnLt, <)
FK_BINARY_FUNCTOR(FnGe, >=)
FK_BINARY_FUNCTOR(FnLe, <=)
FK_BINARY_FUNCTOR(FnAnd, &&)
FK_BINARY_FUNCTOR(FnOr, ||)
FK_BINARY_FUNCTOR(FnBitAnd, &)
FK_BINARY_FUNCTOR(FnBitOr, |)
FK_BINARY_FUNCTOR(FnBitXor, ^)
#undef FK_BINARY_FUNCTOR

template <typename A, typename B>
constexpr bool can_binary = CanBinary<A, B>::value;
template <typename A, typename B>
constexpr bool can_bitwise = CanBinaryBitwise<A, B>::value;
} // namespace detail

} // namespace fk

// The operators live in namespace fk beside the structs, so argument-dependent lookup finds them from any namespace
// (the reference declares its own globally because it operates on the CUDA runtime's global types,
// core/utils/cuda_vector_utils.h:499-602).
#define FK_VEC_OPERATOR(OP, FN, COND)                                                                                  \
    template <typename A, typename B, std::enable_if_t<fk::detail::COND<A, B>, int> = 0>                               \
    FK_HD_CNST auto operator OP(const A& a, const B& b) {                                                              \
        return fk::detail::vec_binary<fk::detail::FN>(a, b);                                                           \
    }
namespace fk {
FK_VEC_OPERATOR(+, FnAdd, can_binary)
FK_VEC_OPERATOR(-, FnSub, can_binary)
FK_VEC_OPERATOR(*, FnMul, can_binary)
FK_VEC_OPERATOR(/, FnDiv, can_binary)
FK_VEC_OPERATOR(==, FnEq, can_binary)
FK_VEC_OPERATOR(!=, FnNe, can_binary)
FK_VEC_OPERATOR(>, FnGt, can_binary)
FK_VEC_OPERATOR(<, FnLt, can_binary)
FK_VEC_OPERATOR(>=, FnGe, can_binary)
FK_VEC_OPERATOR(<=, FnLe, can_binary)
FK_VEC_OPERATOR(&&, FnAnd, can_binary)
FK_VEC_OPERATOR(||, FnOr, can_binary)
FK_VEC_OPERATOR(&, FnBitAnd, can_bitwise)
FK_VEC_OPERATOR(|, FnBitOr, can_bitwise)
FK_VEC_OPERATOR(^, FnBitXor, can_bitwise)

// Unary operators per channel; the result has the base type the scalar expression yields (a one-channel vector gives
// that scalar itself, as in the reference), and an operator the base type does not have is not offered for its vectors.
#define FK_VEC_UNARY(OP)                                                                                               \
    template <typename T, std::enable_if_t<CanUnary<T>::value, int> = 0>                                               \
    FK_HD_CNST auto operator OP(const T& a) -> VectorType_t<decltype(OP std::declval<VBase<T>>()), cn<T>> {            \
        using O = VectorType_t<decltype(OP std::declval<VBase<T>>()), cn<T>>;                                          \
        if constexpr (cn<T> == 1) {                                                                                    \
            return make_<O>(OP a.x);                                                                                   \
        } else if constexpr (cn<T> == 2) {                                                                             \
            return make_<O>(OP a.x, OP a.y);                                                                           \
        } else if constexpr (cn<T> == 3) {                                                                             \
            return make_<O>(OP a.x, OP a.y, OP a.z);                                                                   \
        } else {                                                                                                       \
            return make_<O>(OP a.x, OP a.y, OP a.z, OP a.w);                                                           \
        }                                                                                                              \
    }
FK_VEC_UNARY(-)
FK_VEC_UNARY(!)
FK_VEC_UNARY(~)
#undef FK_VEC_UNARY

// Compound assignment per channel: vector op= vector of the same channel count, or vector op= scalar.
#define FK_VEC_COMPOUND(OP, COND)                                                                                      \
    template <typename I1, typename I2, std::enable_if_t<COND<I1, I2>::value, int> = 0>                                \
    FK_HD_CNST I1 operator OP(I1& a, const I2& b) {                                                                    \
        a.x OP vget<0>(b);                                                                                             \
        if constexpr (cn<I1> >= 2) a.y OP vget<1>(b);                                                                  \
        if constexpr (cn<I1> >= 3) a.z OP vget<2>(b);                                                                  \
        if constexpr (cn<I1> == 4) a.w OP vget<3>(b);                                                                  \
        return a;                                                                                                      \
    }
FK_VEC_COMPOUND(+=, CanCompound)
FK_VEC_COMPOUND(-=, CanCompound)
FK_VEC_COMPOUND(*=, CanCompound)
FK_VEC_COMPOUND(/=, CanCompound)
FK_VEC_COMPOUND(&=, CanCompoundLogical)
FK_VEC_COMPOUND(|=, CanCompoundLogical)
#undef FK_VEC_COMPOUND
} // namespace fk
#undef FK_VEC_OPERATOR

#endif
