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

// A build with FK_INTERPOLATE_Y1_FROM_X takes the bilinear interpolation's upper row index from the x coordinate, as the
// reference's host branch does (interpolation.h:69-70).  Over a window of win_w columns whose first row is row `oy` of an
// image of img_h rows it then reads image rows up to oy + win_w - 1, whatever the window's height: the entry points of
// such a build refuse windows for which those rows do not exist (the read has no bounds check, as in the reference).
inline bool interpolation_rows_exist(int oy, int win_w, int img_h) {
#ifdef FK_INTERPOLATE_Y1_FROM_X
    return oy + win_w <= img_h;
#else
    (void)oy; (void)win_w; (void)img_h;
    return true;
#endif
}
inline int rows_missing() {
    return unsupported("this build takes the interpolation's row index from the x coordinate: a source window may be at most as "
                       "wide as the image has rows from the window's first row on");
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
