// Basic macros, scalar aliases and the runtime error check of the fk:: template layer.
// Counterpart of the reference's core/utils/utils.h:32-152 (function attribute macros, gpuErrchk, NullType).
#ifndef FK_CORE_UTILS_H
#define FK_CORE_UTILS_H

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <utility>

#include "fk_hip_rt.h"

#define FK_HD __host__ __device__ inline
#define FK_HD_CNST __host__ __device__ inline constexpr
#define FK_HD_STATIC __host__ __device__ static inline constexpr
#define FK_D_STATIC __device__ static inline
#define FK_H_STATIC static inline

// The reference spells its attribute macros this way; kept so user operations written against it still compile.
#define FK_HOST_DEVICE_FUSE FK_HD_STATIC
#define FK_HOST_DEVICE_CNST FK_HD_CNST
#define FK_DEVICE_FUSE __device__ static inline constexpr
#define FK_HOST_FUSE static inline constexpr
#define FK_HOST_CNST inline constexpr

// Makes a struct of static members impossible to instantiate (core/utils/utils.h:77-83).
#define FK_STATIC_STRUCT(NAME, SELF)                                                                                  \
    NAME() = delete;                                                                                                   \
    NAME(const SELF&) = delete;                                                                                        \
    NAME(SELF&&) = delete;                                                                                             \
    SELF& operator=(const SELF&) = delete;                                                                             \
    SELF& operator=(SELF&&) = delete;

namespace fk {

using uchar = unsigned char;
using schar = signed char;
using ushort = unsigned short;
using uint = unsigned int;
using ulong = unsigned long;
using longlong = long long;
using ulonglong = unsigned long long;

struct NullType {};

template <typename... Types>
struct TypeList {
    enum { size = sizeof...(Types) };
};
// A TypeList of four or of six TypeLists also names their concatenation as ::type (core/utils/type_lists.h:49-59).
template <typename... A, typename... B, typename... C, typename... D>
struct TypeList<TypeList<A...>, TypeList<B...>, TypeList<C...>, TypeList<D...>> {
    enum { size = 4 };
    using type = TypeList<A..., B..., C..., D...>;
};
template <typename... A, typename... B, typename... C, typename... D, typename... E, typename... F>
struct TypeList<TypeList<A...>, TypeList<B...>, TypeList<C...>, TypeList<D...>, TypeList<E...>, TypeList<F...>> {
    enum { size = 6 };
    using type = TypeList<A..., B..., C..., D..., E..., F...>;
};

// Throws std::runtime_error("GPU Error: <text> File: <file> Line: <line>") on a non-zero runtime status, the
// text convention of the reference's gpuAssert (core/utils/utils.h:95-109).
inline void gpuAssert(int status, const char* file, int line) {
    if (status != 0) {
        throw std::runtime_error(std::string("GPU Error: ") + fkrt_error_string(status) + " File: " + file +
                                 " Line: " + std::to_string(line));
    }
}

} // namespace fk

#define gpuErrchk(status) ::fk::gpuAssert(static_cast<int>(status), __FILE__, __LINE__)

#endif
