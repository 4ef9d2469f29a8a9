// Helpers shared by the translation units of libfk_capi.so: the per-thread error text, the exception guard and
// RawPtr views over caller memory.
#ifndef FK_CAPI_COMMON_H
#define FK_CAPI_COMMON_H

#include <exception>
#include <string>

#include "fk/fused_kernel.h"
#include "fk_capi.h"

namespace fk_capi {

// The text fk_last_error() returns on this thread (defined in fk_capi.hip).
std::string& last_error();

template <typename F>
int guarded(F&& body) {
    try {
        return body();
    } catch (const std::exception& e) {
        last_error() = e.what();
        return FK_ERR_RUNTIME;
    }
}
inline int bad_argument(const char* what) {
    last_error() = what;
    return FK_ERR_ARGUMENT;
}
inline int unsupported(const char* what) {
    last_error() = what;
    return FK_ERR_UNSUPPORTED;
}

template <typename T>
fk::RawPtr<fk::ND::_2D, T> view2d(const void* data, int w, int h, size_t pitch) {
    return fk::RawPtr<fk::ND::_2D, T>{ const_cast<T*>(static_cast<const T*>(data)),
                                       fk::PtrDims<fk::ND::_2D>(static_cast<fk::uint>(w), static_cast<fk::uint>(h), static_cast<fk::uint>(pitch)) };
}
template <typename T>
fk::RawPtr<fk::ND::_3D, T> view3d(void* data, int w, int h, int planes, int color_planes) {
    return fk::RawPtr<fk::ND::_3D, T>{ static_cast<T*>(data),
                                       fk::PtrDims<fk::ND::_3D>(static_cast<fk::uint>(w), static_cast<fk::uint>(h), static_cast<fk::uint>(planes),
                                                                static_cast<fk::uint>(color_planes), static_cast<fk::uint>(sizeof(T) * w)) };
}

} // namespace fk_capi
#endif
