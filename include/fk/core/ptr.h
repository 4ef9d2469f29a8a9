// Owning, reference-counted buffers: Ptr<ND,T>, Ptr1D/2D/3D, Tensor.  Same public surface and error behaviour as
// the reference's core/data/ptr_nd.h:134-714 (MemType, upload/download, crop, at(), getPlane, refcount), with all
// allocation and copies going through the C runtime ABI.  2-D device buffers get the runtime's padded pitch and a
// tight pinned host mirror (ptr_nd.h:68-81,187-201); tensors are tight (ptr_nd.h:85-104,684-685).
#ifndef FK_CORE_PTR_H
#define FK_CORE_PTR_H

#include <atomic>
#include <cstdlib>

#include "fk/core/data.h"
#include "fk/core/stream.h"

namespace fk {

enum class MemType { Device, Host, HostPinned, DeviceAndPinned };
constexpr MemType defaultMemType = MemType::DeviceAndPinned;

struct RefPtr {
    void* ptr{ nullptr };
    void* pinnedPtr{ nullptr };
    std::atomic<int> cnt{ 1 };
};

namespace detail {
template <ND D, typename T>
struct PtrLayout;
template <typename T>
struct PtrLayout<ND::_1D, T> {
    static size_t bytes(const PtrDims<ND::_1D>& d) { return d.pitch; }
    static uint elements(const PtrDims<ND::_1D>& d) { return d.width; }
    static void tight(PtrDims<ND::_1D>& d) { d.pitch = static_cast<uint>(sizeof(T)) * d.width; }
    static size_t rows(const PtrDims<ND::_1D>&) { return 1; }
};
template <typename T>
struct PtrLayout<ND::_2D, T> {
    static size_t bytes(const PtrDims<ND::_2D>& d) { return static_cast<size_t>(d.pitch) * d.height; }
    static uint elements(const PtrDims<ND::_2D>& d) { return d.width * d.height; }
    static void tight(PtrDims<ND::_2D>& d) { d.pitch = static_cast<uint>(sizeof(T)) * d.width; }
    static size_t rows(const PtrDims<ND::_2D>& d) { return d.height; }
};
template <typename T>
struct PtrLayout<ND::_3D, T> {
    static size_t bytes(const PtrDims<ND::_3D>& d) { return static_cast<size_t>(d.pitch) * d.height * d.planes * d.color_planes; }
    static uint elements(const PtrDims<ND::_3D>& d) { return d.width * d.height * d.planes * d.color_planes; }
    static void tight(PtrDims<ND::_3D>& d) {
        d.pitch = static_cast<uint>(sizeof(T)) * d.width;
        d.plane_pitch = d.pitch * d.height;
    }
    static size_t rows(const PtrDims<ND::_3D>& d) { return static_cast<size_t>(d.height) * d.planes * d.color_planes; }
};
template <typename T>
struct PtrLayout<ND::T3D, T> {
    static size_t bytes(const PtrDims<ND::T3D>& d) { return static_cast<size_t>(d.color_planes_pitch) * d.color_planes; }
    static uint elements(const PtrDims<ND::T3D>& d) { return d.width * d.height * d.planes * d.color_planes; }
    static void tight(PtrDims<ND::T3D>& d) {
        d.pitch = static_cast<uint>(sizeof(T)) * d.width;
        d.plane_pitch = d.pitch * d.height;
        d.color_planes_pitch = d.plane_pitch * d.planes;
    }
    static size_t rows(const PtrDims<ND::T3D>& d) { return static_cast<size_t>(d.height) * d.planes * d.color_planes; }
};
} // namespace detail

template <ND D, typename T>
class Ptr {
    using Layout = detail::PtrLayout<D, T>;

protected:
    RefPtr* ref{ nullptr };
    RawPtr<D, T> ptr_a;      // device view (or the only view for single-space buffers)
    RawPtr<D, T> ptr_pinned; // host view
    MemType type{ defaultMemType };
    int deviceID{ 0 };

    void release() {
        if (ref != nullptr && ref->cnt.fetch_sub(1) == 1) {
            switch (type) {
            case MemType::Device: (void)fkrt_free(ref->ptr); break;
            case MemType::Host: std::free(ref->ptr); break;
            case MemType::HostPinned: (void)fkrt_free_host(ref->ptr); break;
            case MemType::DeviceAndPinned:
                (void)fkrt_free(ref->ptr);
                (void)fkrt_free_host(ref->pinnedPtr);
                break;
            }
            delete ref;
        }
        ref = nullptr;
    }
    void shareFrom(const Ptr& other) {
        ref = other.ref;
        ptr_a = other.ptr_a;
        ptr_pinned = other.ptr_pinned;
        type = other.type;
        deviceID = other.deviceID;
        if (ref != nullptr) ref->cnt.fetch_add(1);
    }
    void allocDeviceSide(bool honour_given_pitch) {
        int current = 0;
        gpuErrchk(fkrt_get_device(&current));
        gpuErrchk(fkrt_set_device(deviceID));
        void* p = nullptr;
        if constexpr (D == ND::_2D) {
            if (honour_given_pitch && ptr_a.dims.pitch != 0) {
                gpuErrchk(fkrt_malloc(&p, Layout::bytes(ptr_a.dims)));
            } else {
                size_t pitch = 0;
                gpuErrchk(fkrt_malloc_pitch(&p, &pitch, sizeof(T) * ptr_a.dims.width, ptr_a.dims.height));
                ptr_a.dims.pitch = static_cast<uint>(pitch);
            }
        } else {
            if (!(honour_given_pitch && ptr_a.dims.pitch != 0)) Layout::tight(ptr_a.dims);
            gpuErrchk(fkrt_malloc(&p, Layout::bytes(ptr_a.dims)));
        }
        ptr_a.data = static_cast<T*>(p);
        if (current != deviceID) gpuErrchk(fkrt_set_device(current));
    }

public:
    Ptr() {}
    Ptr(const Ptr& other) { shareFrom(other); }
    Ptr(Ptr&& other) noexcept
        : ref(other.ref), ptr_a(other.ptr_a), ptr_pinned(other.ptr_pinned), type(other.type), deviceID(other.deviceID) {
        other.ref = nullptr;
    }
    Ptr& operator=(const Ptr& other) {
        if (this != &other) {
            release();
            shareFrom(other);
        }
        return *this;
    }
    Ptr& operator=(Ptr&& other) noexcept {
        if (this != &other) {
            release();
            ref = other.ref;
            ptr_a = other.ptr_a;
            ptr_pinned = other.ptr_pinned;
            type = other.type;
            deviceID = other.deviceID;
            other.ref = nullptr;
        }
        return *this;
    }
    ~Ptr() { release(); }

    Ptr(const PtrDims<D>& dims, const MemType& type_ = defaultMemType, const int& deviceID_ = 0) { allocPtr(dims, type_, deviceID_); }
    // Allocation by extent, one form per dimensionality (core/data/ptr_nd.h:303-320).
    template <ND DN = D, std::enable_if_t<DN == ND::_1D, int> = 0>
    Ptr(const uint& num_elems, const uint& size_in_bytes = 0, const MemType& type_ = defaultMemType, const int& deviceID_ = 0) {
        allocPtr(PtrDims<ND::_1D>(num_elems, size_in_bytes), type_, deviceID_);
    }
    template <ND DN = D, std::enable_if_t<DN == ND::_2D, int> = 0>
    Ptr(const uint& width_, const uint& height_, const uint& pitch_ = 0, const MemType& type_ = defaultMemType, const int& deviceID_ = 0) {
        allocPtr(PtrDims<ND::_2D>(width_, height_, pitch_), type_, deviceID_);
    }
    template <ND DN = D, std::enable_if_t<DN == ND::_3D, int> = 0>
    Ptr(const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1, const uint& pitch_ = 0,
        const MemType& type_ = defaultMemType, const int& deviceID_ = 0) {
        allocPtr(PtrDims<ND::_3D>(width_, height_, planes_, color_planes_, pitch_), type_, deviceID_);
    }

    // Non-owning views over memory the caller manages.
    Ptr(T* data_, const PtrDims<D>& dims, const MemType& type_, const int& deviceID_) {
        if (type_ == MemType::DeviceAndPinned) {
            throw std::runtime_error("DeviceAndPinned type requires an additional argument for the pinned pointer.");
        }
        ptr_a.data = data_;
        ptr_a.dims = dims;
        ptr_pinned = ptr_a;
        type = type_;
        deviceID = deviceID_;
    }
    Ptr(const RawPtr<D, T>& data_, const MemType& type_, const int& deviceID_) : Ptr(data_.data, data_.dims, type_, deviceID_) {}
    Ptr(T* data_, T* pinned_data, const PtrDims<D>& dims, const MemType& type_, const int& deviceID_) {
        ptr_a.data = data_;
        ptr_a.dims = dims;
        ptr_pinned.data = pinned_data;
        ptr_pinned.dims = dims;
        type = type_;
        deviceID = deviceID_;
    }

    void allocPtr(const PtrDims<D>& dims_, const MemType& type_ = defaultMemType, const int& deviceID_ = 0) {
        if (ref != nullptr) {
            throw std::runtime_error("Reference pointer already exists. Use a different constructor.");
        }
        ptr_a.dims = dims_;
        ptr_pinned.dims = dims_;
        type = type_;
        deviceID = deviceID_;
        ref = new RefPtr();
        switch (type) {
        case MemType::Device:
            allocDeviceSide(true);
            ptr_pinned = ptr_a;
            break;
        case MemType::Host: {
            if (ptr_a.dims.pitch == 0) Layout::tight(ptr_a.dims);
            ptr_a.data = static_cast<T*>(std::malloc(Layout::bytes(ptr_a.dims)));
            if (ptr_a.data == nullptr) throw std::runtime_error("Host allocation failed.");
            ptr_pinned = ptr_a;
            break;
        }
        case MemType::HostPinned: {
            if (ptr_a.dims.pitch == 0) Layout::tight(ptr_a.dims);
            void* p = nullptr;
            gpuErrchk(fkrt_malloc_host(&p, Layout::bytes(ptr_a.dims)));
            ptr_a.data = static_cast<T*>(p);
            ptr_pinned = ptr_a;
            break;
        }
        case MemType::DeviceAndPinned: {
            allocDeviceSide(true);
            Layout::tight(ptr_pinned.dims);
            void* p = nullptr;
            gpuErrchk(fkrt_malloc_host(&p, Layout::bytes(ptr_pinned.dims)));
            ptr_pinned.data = static_cast<T*>(p);
            break;
        }
        }
        ref->ptr = ptr_a.data;
        ref->pinnedPtr = ptr_pinned.data;
    }

    RawPtr<D, T> ptr() const { return ptr_a; }
    RawPtr<D, T> ptrPinned() const { return ptr_pinned; }
    operator RawPtr<D, T>() const { return ptr_a; }
    PtrDims<D> dims() const { return ptr_a.dims; }
    MemType getMemType() const { return type; }
    int getDeviceID() const { return deviceID; }
    size_t sizeInBytes() const { return Layout::bytes(ptr_a.dims); }
    uint getNumElements() const { return Layout::elements(ptr_a.dims); }
    int getRefCount() const { return ref != nullptr ? ref->cnt.load() : 0; }

    // A view of a sub-rectangle that shares ownership with this buffer (ptr_nd.h:410-423).
    Ptr<D, T> crop(const Point& p, const PtrDims<D>& newDims) {
        Ptr<D, T> view(*this);
        view.ptr_a.data = PtrAccessor<D>::point(p, ptr_a);
        view.ptr_a.dims = newDims;
        view.ptr_a.dims.pitch = ptr_a.dims.pitch;
        view.ptr_pinned.data = PtrAccessor<D>::point(p, ptr_pinned);
        view.ptr_pinned.dims = newDims;
        view.ptr_pinned.dims.pitch = ptr_pinned.dims.pitch;
        if constexpr (D == ND::_3D) {
            view.ptr_a.dims.plane_pitch = ptr_a.dims.plane_pitch;
            view.ptr_pinned.dims.plane_pitch = ptr_pinned.dims.plane_pitch;
        }
        return view;
    }

private:
    static bool onDevice(MemType t) { return t == MemType::Device || t == MemType::DeviceAndPinned; }
    static void copyRaw(const RawPtr<D, T>& from, const RawPtr<D, T>& to, int kind, fkrt_stream stream) {
        const size_t row_bytes = sizeof(T) * from.dims.width;
        if (from.dims.pitch == to.dims.pitch) {
            gpuErrchk(fkrt_memcpy_async(to.data, from.data, Layout::bytes(from.dims), kind, stream));
        } else {
            gpuErrchk(fkrt_memcpy2d_async(to.data, to.dims.pitch, from.data, from.dims.pitch, row_bytes,
                                          Layout::rows(from.dims), kind, stream));
        }
    }
    static bool sameShape(const PtrDims<D>& a, const PtrDims<D>& b) {
        if constexpr (D == ND::_1D) return a.width == b.width;
        else if constexpr (D == ND::_2D) return a.width == b.width && a.height == b.height;
        else return a.width == b.width && a.height == b.height && a.planes == b.planes && a.color_planes == b.color_planes;
    }

public:
    // Host-side buffer -> device buffer `other`.
    void uploadTo(Ptr<D, T>& other, fkrt_stream stream = nullptr) {
        if (type == MemType::Device) throw std::runtime_error("Upload can only be performed from Host, HostPinned or DeviceAndPinned memory.");
        if (!onDevice(other.type)) throw std::runtime_error("Upload destination must be Device or DeviceAndPinned memory.");
        if (!sameShape(ptr_pinned.dims, other.ptr_a.dims)) throw std::runtime_error("Size mismatch between source and destination.");
        copyRaw(ptr_pinned, other.ptr_a, FKRT_H2D, stream);
    }
    // Device buffer -> host-side buffer `other`.
    void downloadTo(Ptr<D, T>& other, fkrt_stream stream = nullptr) {
        if (!onDevice(type)) throw std::runtime_error("Download can only be performed from Device or DeviceAndPinned memory.");
        if (other.type == MemType::Device) throw std::runtime_error("Download destination must be Host, HostPinned or DeviceAndPinned memory.");
        if (!sameShape(ptr_a.dims, other.ptr_pinned.dims)) throw std::runtime_error("Size mismatch between source and destination.");
        copyRaw(ptr_a, other.ptr_pinned, FKRT_D2H, stream);
    }
    // Between the two halves of a DeviceAndPinned buffer; no-ops for single-space buffers.
    void upload(Stream& stream) {
        if (type == MemType::DeviceAndPinned) copyRaw(ptr_pinned, ptr_a, FKRT_H2D, stream.getHIPStream());
    }
    void download(Stream& stream) {
        if (type == MemType::DeviceAndPinned) copyRaw(ptr_a, ptr_pinned, FKRT_D2H, stream.getHIPStream());
    }

    // Host access (pinned mirror or host buffer); device-only memory throws (ptr_nd.h:537-588).
    T& at(const Point& p) {
        if (type == MemType::Device) throw std::runtime_error("This is a device pointer, cannot access data with at().");
        return *PtrAccessor<D>::point(p, ptr_pinned);
    }
    T at(const Point& p) const {
        if (type == MemType::Device) throw std::runtime_error("This is a device pointer, cannot access data with at().");
        return *PtrAccessor<D>::cr_point(p, ptr_pinned);
    }
    T& at(const uint& x) { return at(Point(static_cast<int>(x))); }
    T at(const uint& x) const { return at(Point(static_cast<int>(x))); }
    template <ND DIM = D, std::enable_if_t<DIM == ND::_2D || DIM == ND::_3D, int> = 0>
    T& at(const uint& x, const uint& y) { return at(Point(static_cast<int>(x), static_cast<int>(y))); }
    template <ND DIM = D, std::enable_if_t<DIM == ND::_2D || DIM == ND::_3D, int> = 0>
    T at(const uint& x, const uint& y) const { return at(Point(static_cast<int>(x), static_cast<int>(y))); }
    template <ND DIM = D, std::enable_if_t<DIM == ND::_3D || DIM == ND::T3D, int> = 0>
    T& at(const uint& x, const uint& y, const uint& z) { return at(Point(static_cast<int>(x), static_cast<int>(y), static_cast<int>(z))); }
    template <ND DIM = D, std::enable_if_t<DIM == ND::_3D || DIM == ND::T3D, int> = 0>
    T at(const uint& x, const uint& y, const uint& z) const { return at(Point(static_cast<int>(x), static_cast<int>(y), static_cast<int>(z))); }

    // One image of a 3-D buffer as a 2-D buffer sharing ownership (ptr_nd.h:590-601).
    template <ND DIM = D, std::enable_if_t<DIM == ND::_3D, int> = 0>
    Ptr<ND::_2D, T> getPlane(const uint& plane) {
        if (plane >= ptr_a.dims.planes) throw std::runtime_error("Plane index out of range.");
        const PtrDims<ND::_2D> d2(ptr_a.dims.width, ptr_a.dims.height * ptr_a.dims.color_planes, ptr_a.dims.pitch);
        T* const dev = PtrAccessor<ND::_3D>::point(Point(0, 0, static_cast<int>(plane)), ptr_a);
        T* const host = PtrAccessor<ND::_3D>::point(Point(0, 0, static_cast<int>(plane)), ptr_pinned);
        PtrDims<ND::_2D> h2 = d2;
        h2.pitch = ptr_pinned.dims.pitch;
        return Ptr<ND::_2D, T>::makeView(ref, dev, d2, host, h2, type, deviceID);
    }

    static Ptr makeView(RefPtr* ref_, T* dev, const PtrDims<D>& ddims, T* host, const PtrDims<D>& hdims, MemType type_, int dev_id) {
        Ptr v;
        v.ref = ref_;
        if (ref_ != nullptr) ref_->cnt.fetch_add(1);
        v.ptr_a.data = dev;
        v.ptr_a.dims = ddims;
        v.ptr_pinned.data = host;
        v.ptr_pinned.dims = hdims;
        v.type = type_;
        v.deviceID = dev_id;
        return v;
    }
};

template <typename T>
class Ptr1D : public Ptr<ND::_1D, T> {
public:
    Ptr1D() {}
    Ptr1D(const uint& num_elems, const uint& size_in_bytes = 0, const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::_1D, T>(PtrDims<ND::_1D>(num_elems, size_in_bytes), type_, deviceID_) {}
    Ptr1D(const Ptr<ND::_1D, T>& other) : Ptr<ND::_1D, T>(other) {}
    Ptr1D(T* data_, const PtrDims<ND::_1D>& dims_, const MemType& type_ = MemType::Device, const int& deviceID_ = 0)
        : Ptr<ND::_1D, T>(data_, dims_, type_, deviceID_) {}
    Ptr1D<T> crop1D(const Point& p, const PtrDims<ND::_1D>& newDims) { return Ptr<ND::_1D, T>::crop(p, newDims); }
};

template <typename T>
class Ptr2D : public Ptr<ND::_2D, T> {
public:
    Ptr2D() {}
    Ptr2D(const Size& size, const uint& pitch_ = 0, const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::_2D, T>(PtrDims<ND::_2D>(size.width, size.height, pitch_), type_, deviceID_) {}
    Ptr2D(const uint& width_, const uint& height_, const uint& pitch_ = 0, const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::_2D, T>(PtrDims<ND::_2D>(width_, height_, pitch_), type_, deviceID_) {}
    Ptr2D(const Ptr<ND::_2D, T>& other) : Ptr<ND::_2D, T>(other) {}
    Ptr2D(T* data_, const uint& width_, const uint& height_, const uint& pitch_, const MemType& type_ = MemType::Device, const int& deviceID_ = 0)
        : Ptr<ND::_2D, T>(data_, PtrDims<ND::_2D>(width_, height_, pitch_), type_, deviceID_) {}
    Ptr2D<T> crop2D(const Point& p, const PtrDims<ND::_2D>& newDims) { return Ptr<ND::_2D, T>::crop(p, newDims); }
    void Alloc(const Size& size, const uint& pitch_ = 0, const MemType& type_ = defaultMemType, const int& deviceID_ = 0) {
        this->allocPtr(PtrDims<ND::_2D>(size.width, size.height, pitch_), type_, deviceID_);
    }
};

template <typename T>
class Ptr3D : public Ptr<ND::_3D, T> {
public:
    Ptr3D(const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1, const uint& pitch_ = 0,
          const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::_3D, T>(PtrDims<ND::_3D>(width_, height_, planes_, color_planes_, pitch_), type_, deviceID_) {}
    Ptr3D(const Ptr<ND::_3D, T>& other) : Ptr<ND::_3D, T>(other) {}
    Ptr3D(T* data_, const PtrDims<ND::_3D>& dims_, const MemType& type_ = MemType::Device, const int& deviceID_ = 0)
        : Ptr<ND::_3D, T>(data_, dims_, type_, deviceID_) {}
    Ptr3D<T> crop3D(const Point& p, const PtrDims<ND::_3D>& newDims) { return Ptr<ND::_3D, T>::crop(p, newDims); }
};

// A 3D pointer whose channel planes are outermost (ptr_nd.h:661-675).
template <typename T>
class PtrT3D : public Ptr<ND::T3D, T> {
public:
    PtrT3D(const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1, const MemType& type_ = defaultMemType,
           const int& deviceID_ = 0)
        : Ptr<ND::T3D, T>(PtrDims<ND::T3D>(width_, height_, planes_, color_planes_), type_, deviceID_) {}
    PtrT3D(const Ptr<ND::T3D, T>& other) : Ptr<ND::T3D, T>(other) {}
    PtrT3D(T* data_, const PtrDims<ND::T3D>& dims_, const MemType& type_ = MemType::Device, const int& deviceID_ = 0)
        : Ptr<ND::T3D, T>(data_, dims_, type_, deviceID_) {}
    PtrT3D<T> crop3D(const Point& p, const PtrDims<ND::T3D>& newDims) { return Ptr<ND::T3D, T>::crop(p, newDims); }
};

// width x height x planes images of `color_planes` channel planes each, rows always tight.
template <typename T>
class Tensor : public Ptr<ND::_3D, T> {
public:
    Tensor() {}
    Tensor(const Tensor<T>& other) : Ptr<ND::_3D, T>(other) {}
    Tensor(const Ptr<ND::_3D, T>& other) : Ptr<ND::_3D, T>(other) {}
    Tensor(const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1,
           const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::_3D, T>(PtrDims<ND::_3D>(width_, height_, planes_, color_planes_, static_cast<uint>(sizeof(T)) * width_), type_, deviceID_) {}
    Tensor(T* data, const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1,
           const MemType& type_ = MemType::Device, const int& deviceID_ = 0)
        : Ptr<ND::_3D, T>(data, PtrDims<ND::_3D>(width_, height_, planes_, color_planes_, static_cast<uint>(sizeof(T)) * width_), type_, deviceID_) {}
    Tensor& operator=(const Tensor&) = default;
    void allocTensor(const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1,
                     const MemType& type_ = defaultMemType, const int& deviceID_ = 0) {
        this->allocPtr(PtrDims<ND::_3D>(width_, height_, planes_, color_planes_, static_cast<uint>(sizeof(T)) * width_), type_, deviceID_);
    }
};

// A tensor whose channel planes are outermost: element (x, y, z) of channel c at
// c*color_planes_pitch + z*plane_pitch + y*pitch + x (ptr_nd.h:104-126,696-714).
template <typename T>
class TensorT : public Ptr<ND::T3D, T> {
public:
    TensorT() {}
    TensorT(const TensorT<T>& other) : Ptr<ND::T3D, T>(other) {}
    TensorT(const Ptr<ND::T3D, T>& other) : Ptr<ND::T3D, T>(other) {}
    TensorT(const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1,
            const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::T3D, T>(tightDims(width_, height_, planes_, color_planes_), type_, deviceID_) {}
    TensorT(T* data, const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1,
            const MemType& type_ = MemType::Device, const int& deviceID_ = 0)
        : Ptr<ND::T3D, T>(data, tightDims(width_, height_, planes_, color_planes_), type_, deviceID_) {}
    TensorT& operator=(const TensorT&) = default;
    void allocTensor(const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1,
                     const MemType& type_ = defaultMemType, const int& deviceID_ = 0) {
        this->allocPtr(tightDims(width_, height_, planes_, color_planes_), type_, deviceID_);
    }

private:
    static PtrDims<ND::T3D> tightDims(uint w, uint h, uint planes, uint color_planes) {
        PtrDims<ND::T3D> d(w, h, planes, color_planes);
        detail::PtrLayout<ND::T3D, T>::tight(d);
        return d;
    }
};

} // namespace fk
#endif
