// Geometry and non-owning pointer types: ND, Point, Size, Rect, ActiveThreads, PtrDims, RawPtr, PtrAccessor.
// Same fields and meaning as the reference's core/data/{nd,point,size,rect,rawptr}.h and
// core/execution_model/active_threads.h:25-33; addressing follows core/data/rawptr.h:186-239.
#ifndef FK_CORE_DATA_H
#define FK_CORE_DATA_H

#include "fk/core/vector_types.h"

namespace fk {

enum class ND { _1D = 1, _2D = 2, _3D = 3, T3D = 4 };

template <typename T, ND D>
struct Point_;
template <typename T>
struct Point_<T, ND::_1D> {
    T x;
    FK_HD_CNST Point_(const T x_ = 0) : x(x_) {}
};
template <typename T>
struct Point_<T, ND::_2D> {
    T x, y;
    FK_HD_CNST Point_(const T x_ = 0, const T y_ = 0) : x(x_), y(y_) {}
};
template <typename T>
struct Point_<T, ND::_3D> {
    T x, y, z;
    FK_HD_CNST Point_(const T x_ = 0, const T y_ = 0, const T z_ = 0) : x(x_), y(y_), z(z_) {}
};
using Point = Point_<int, ND::_3D>;

template <typename T>
struct Size_ {
    T width{ 0 };
    T height{ 0 };
    FK_HD_CNST Size_() {}
    FK_HD_CNST Size_(T width_, T height_) : width(width_), height(height_) {}
};
using Size = Size_<int>;

template <typename P, typename S = P>
struct Rect_ {
    P x{ 0 }, y{ 0 };
    S width{ 0 }, height{ 0 };
    FK_HD_CNST Rect_() {}
    FK_HD_CNST Rect_(const Point& point, const Size& size) : x(point.x), y(point.y), width(size.width), height(size.height) {}
    FK_HD_CNST Rect_(const P& x_, const P& y_, const S& width_, const S& height_) : x(x_), y(y_), width(width_), height(height_) {}
};
using Rect = Rect_<uint, int>;

struct ActiveThreads {
    uint x{ 1 }, y{ 1 }, z{ 1 };
    FK_HD_CNST ActiveThreads() {}
    FK_HD_CNST ActiveThreads(const uint& vx, const uint& vy = 1, const uint& vz = 1) : x(vx), y(vy), z(vz) {}
    FK_HD_CNST bool operator==(const ActiveThreads& o) const { return x == o.x && y == o.y && z == o.z; }
};

template <ND D>
struct PtrDims;
template <>
struct PtrDims<ND::_1D> {
    uint width{ 0 };
    uint pitch{ 0 };
    FK_HD_CNST PtrDims() {}
    FK_HD_CNST PtrDims(uint width_, uint pitch_ = 0) : width(width_), pitch(pitch_) {}
};
template <>
struct PtrDims<ND::_2D> {
    uint width{ 0 };
    uint height{ 0 };
    uint pitch{ 0 }; // bytes between rows
    FK_HD_CNST PtrDims() {}
    FK_HD_CNST PtrDims(uint width_, uint height_, uint pitch_ = 0) : width(width_), height(height_), pitch(pitch_) {}
};
template <>
struct PtrDims<ND::_3D> {
    uint width{ 0 };
    uint height{ 0 };
    uint planes{ 0 };       // number of images
    uint color_planes{ 0 }; // channel planes per image (1 for packed pixels)
    uint pitch{ 0 };        // bytes between rows
    uint plane_pitch{ 0 };  // bytes between channel planes
    FK_HD_CNST PtrDims() {}
    FK_HD_CNST PtrDims(uint width_, uint height_, uint planes_, uint color_planes_ = 1, uint pitch_ = 0)
        : width(width_), height(height_), planes(planes_), color_planes(color_planes_), pitch(pitch_),
          plane_pitch(pitch_ * height_) {}
};
template <>
struct PtrDims<ND::T3D> {
    uint width{ 0 };
    uint height{ 0 };
    uint planes{ 0 };
    uint color_planes{ 0 };
    uint pitch{ 0 };
    uint plane_pitch{ 0 };
    uint color_planes_pitch{ 0 };
    FK_HD_CNST PtrDims() {}
    FK_HD_CNST PtrDims(uint width_, uint height_, uint planes_, uint color_planes_ = 1)
        : width(width_), height(height_), planes(planes_), color_planes(color_planes_) {}
};

template <ND D, typename T>
struct RawPtr {
    T* data{ nullptr };
    PtrDims<D> dims;
    using type = T;
    enum { ND = static_cast<int>(D) };
};

// Small fixed-size arrays carried by value inside operation parameters (core/data/rawptr.h:106-184): data[H][W].
template <int W>
struct StaticPtrDims1D {
    static constexpr uint width{ W };
};
template <int W, int H>
struct StaticPtrDims2D {
    static constexpr uint width{ W };
    static constexpr uint height{ H };
};
template <int W, int H, int P>
struct StaticPtrDims3D {
    static constexpr uint width{ W };
    static constexpr uint height{ H };
    static constexpr uint planes{ P };
};
template <typename Dims, typename T>
struct StaticRawPtr;
template <typename T, int W>
struct StaticRawPtr<StaticPtrDims1D<W>, T> {
    using type = T;
    T data[W];
    static constexpr StaticPtrDims1D<W> dims{};
    static constexpr ND NDim{ ND::_1D };
};
template <typename T, int W, int H>
struct StaticRawPtr<StaticPtrDims2D<W, H>, T> {
    using type = T;
    T data[H][W];
    static constexpr StaticPtrDims2D<W, H> dims{};
    static constexpr ND NDim{ ND::_2D };
};
template <typename T, int W, int H, int P>
struct StaticRawPtr<StaticPtrDims3D<W, H, P>, T> {
    using type = T;
    T data[P][H][W];
    static constexpr StaticPtrDims3D<W, H, P> dims{};
    static constexpr ND NDim{ ND::_3D };
};

// Byte-pitch addressing of a RawPtr (core/data/rawptr.h:186-239).
template <ND D>
struct PtrAccessor;
template <>
struct PtrAccessor<ND::_1D> {
    template <typename T>
    FK_HD_STATIC T* point(const Point& p, const RawPtr<ND::_1D, T>& ptr) { return ptr.data + p.x; }
    template <typename T>
    FK_HD_STATIC const T* cr_point(const Point& p, const RawPtr<ND::_1D, T>& ptr) { return ptr.data + p.x; }
};
template <>
struct PtrAccessor<ND::_2D> {
    template <typename T>
    FK_HD_STATIC T* point(const Point& p, const RawPtr<ND::_2D, T>& ptr) {
        return reinterpret_cast<T*>(reinterpret_cast<char*>(ptr.data) + static_cast<size_t>(p.y) * ptr.dims.pitch) + p.x;
    }
    template <typename T>
    FK_HD_STATIC const T* cr_point(const Point& p, const RawPtr<ND::_2D, T>& ptr) { return point(p, ptr); }
};
template <>
struct PtrAccessor<ND::_3D> {
    template <typename T>
    FK_HD_STATIC T* point(const Point& p, const RawPtr<ND::_3D, T>& ptr) {
        return reinterpret_cast<T*>(reinterpret_cast<char*>(ptr.data) +
                                    static_cast<size_t>(ptr.dims.plane_pitch) * ptr.dims.color_planes * p.z +
                                    static_cast<size_t>(p.y) * ptr.dims.pitch) + p.x;
    }
    template <typename T>
    FK_HD_STATIC const T* cr_point(const Point& p, const RawPtr<ND::_3D, T>& ptr) { return point(p, ptr); }
};
template <>
struct PtrAccessor<ND::T3D> {
    template <typename T>
    FK_HD_STATIC T* point(const Point& p, const RawPtr<ND::T3D, T>& ptr, const uint& color_plane = 0) {
        return reinterpret_cast<T*>(reinterpret_cast<char*>(ptr.data) +
                                    static_cast<size_t>(color_plane) * ptr.dims.color_planes_pitch +
                                    static_cast<size_t>(ptr.dims.plane_pitch) * p.z +
                                    static_cast<size_t>(ptr.dims.pitch) * p.y) + p.x;
    }
    template <typename T>
    FK_HD_STATIC const T* cr_point(const Point& p, const RawPtr<ND::T3D, T>& ptr, const uint& color_plane = 0) {
        return point(p, ptr, color_plane);
    }
};

namespace detail {
// The element at `p`.  On the GPU a pixel of three one-byte channels is fetched with one (unaligned) dword load instead of
// three byte loads: a wave's memory instructions cost the same address-processing time whatever their width, and kernels
// that gather such pixels one by one are bound by exactly that.  The dword is [p, p + 4) when p is dword-aligned and
// [p - 1, p + 3) otherwise; either way its one byte that is not the pixel's lies in an aligned dword that also holds a
// byte of the pixel, so it is on the pixel's own page: the load cannot fault wherever the buffer begins or ends, and it
// needs no branch, so the taps of an interpolation are in flight together.
template <typename T>
FK_HD_CNST T read_element(const T* p) {
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (validCUDAVec<T> && cn<T> == 3 && sizeof(T) == 3) {
        if (!__builtin_is_constant_evaluated()) {
            using B = VBase<T>;
            const unsigned char* const bytes = reinterpret_cast<const unsigned char*>(p);
            const unsigned back = (static_cast<unsigned>(reinterpret_cast<size_t>(bytes)) & 3u) != 0u ? 1u : 0u;
            unsigned int w = 0;
            __builtin_memcpy(&w, bytes - back, 4);
            w >>= 8u * back;
            return T{ static_cast<B>(static_cast<unsigned char>(w)), static_cast<B>(static_cast<unsigned char>(w >> 8)),
                      static_cast<B>(static_cast<unsigned char>(w >> 16)) };
        }
    }
#endif
    return *p;
}
} // namespace detail

} // namespace fk
#endif
