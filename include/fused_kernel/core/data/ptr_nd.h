// Ptr<D,T>: shared owner of image / tensor memory (device, host, pinned host, or device + pinned mirror), with
// Ptr1D / Ptr2D / Ptr3D / Tensor conveniences.  Interface counterpart: FK/core/data/ptr_nd.h:29-717.
// All device work goes through the C ABI (fklhip_malloc*, fklhip_memcpy*_async); the host never sees a HIP type.
#ifndef FK_AMD_PTR_ND_H
#define FK_AMD_PTR_ND_H

#include <atomic>
#include <cstdlib>
#include <stdexcept>
#include <vector>
#include <type_traits>

#include <fused_kernel/core/data/rawptr.h>
#include <fused_kernel/core/data/size.h>
#include <fused_kernel/core/execution_model/stream.h>
#include <fused_kernel/core/utils/vector_utils.h>

namespace fk {

enum class MemType { Device, Host, HostPinned, DeviceAndPinned };
// GPU builds of the reference default to a device buffer with a pinned host mirror; so does this backend.
constexpr MemType defaultMemType = MemType::DeviceAndPinned;

namespace ptr_detail {

template <ND D, typename T> struct Layout;

template <typename T> struct Layout<ND::_1D, T> {
    static size_t bytes(const PtrDims<ND::_1D>& d) { return d.pitch; }
    static uint elements(const PtrDims<ND::_1D>& d) { return d.width; }
    static void tight(PtrDims<ND::_1D>& d) { if (d.pitch == 0) d.pitch = uint(sizeof(T)) * d.width; }
    static void device_alloc(RawPtr<ND::_1D, T>& p) {
        tight(p.dims);
        gpuErrchk(fklhip_malloc(reinterpret_cast<void**>(&p.data), bytes(p.dims)));
    }
};

template <typename T> struct Layout<ND::_2D, T> {
    static size_t bytes(const PtrDims<ND::_2D>& d) { return size_t(d.pitch) * d.height; }
    static uint elements(const PtrDims<ND::_2D>& d) { return d.width * d.height; }
    static void tight(PtrDims<ND::_2D>& d) { if (d.pitch == 0) d.pitch = uint(sizeof(T)) * d.width; }
    static void device_alloc(RawPtr<ND::_2D, T>& p) {
        if (p.dims.pitch == 0) {
            // pitched allocation: the runtime pads rows to its preferred alignment
            size_t pitch = 0;
            gpuErrchk(fklhip_malloc_pitch(reinterpret_cast<void**>(&p.data), &pitch, sizeof(T) * p.dims.width, p.dims.height));
            p.dims.pitch = uint(pitch);
        } else {
            gpuErrchk(fklhip_malloc(reinterpret_cast<void**>(&p.data), bytes(p.dims)));
        }
    }
};

template <typename T> struct Layout<ND::_3D, T> {
    static size_t bytes(const PtrDims<ND::_3D>& d) { return size_t(d.pitch) * d.height * d.planes * d.color_planes; }
    static uint elements(const PtrDims<ND::_3D>& d) { return d.width * d.height * d.planes * d.color_planes; }
    static void tight(PtrDims<ND::_3D>& d) {
        if (d.pitch == 0) d.pitch = uint(sizeof(T)) * d.width;
        d.plane_pitch = d.pitch * d.height;
    }
    static void device_alloc(RawPtr<ND::_3D, T>& p) {
        tight(p.dims);
        gpuErrchk(fklhip_malloc(reinterpret_cast<void**>(&p.data), bytes(p.dims)));
    }
};

template <typename T> struct Layout<ND::T3D, T> {
    static size_t bytes(const PtrDims<ND::T3D>& d) { return size_t(d.color_planes_pitch) * d.color_planes; }
    static uint elements(const PtrDims<ND::T3D>& d) { return d.width * d.height * d.planes * d.color_planes; }
    static void tight(PtrDims<ND::T3D>& d) {
        if (d.pitch == 0) d.pitch = uint(sizeof(T)) * d.width;
        d.plane_pitch = d.pitch * d.height;
        d.color_planes_pitch = d.plane_pitch * d.planes;
    }
    static void device_alloc(RawPtr<ND::T3D, T>& p) {
        tight(p.dims);
        gpuErrchk(fklhip_malloc(reinterpret_cast<void**>(&p.data), bytes(p.dims)));
    }
};

struct Owner {
    void* ptr{nullptr};
    void* pinnedPtr{nullptr};
    std::atomic<int> cnt{1};
};

// Runs `body` with `device` current and restores the previous device afterwards.
template <typename F> void on_device(int device, F body) {
    int current = 0;
    gpuErrchk(fklhip_get_device(&current));
    if (current != device) gpuErrchk(fklhip_set_device(device));
    try { body(); } catch (...) { if (current != device) fklhip_set_device(current); throw; }
    if (current != device) gpuErrchk(fklhip_set_device(current));
}

} // namespace ptr_detail

using RefPtr = ptr_detail::Owner;

template <ND D, typename T> class Ptr {
public:
    using Type = T;
    using At = PtrAccessor<D>;
    static constexpr ND nd = D;

protected:
    using L = ptr_detail::Layout<D, T>;
    RefPtr* ref{nullptr};
    RawPtr<D, T> ptr_a{};
    RawPtr<D, T> ptr_pinned{};
    MemType type{defaultMemType};
    int deviceID{0};

    void retain() { if (ref) ref->cnt.fetch_add(1); }

    void freePtr() {
        if (!ref) return;
        if (ref->cnt.load() < 1) throw std::runtime_error("Reference count is less than 1, cannot free memory.");
        if (ref->cnt.fetch_sub(1) == 1) {
            switch (type) {
            case MemType::Device: gpuErrchk(fklhip_free(ref->ptr)); break;
            case MemType::Host: std::free(ref->ptr); break;
            case MemType::HostPinned: gpuErrchk(fklhip_host_free(ref->ptr)); break;
            case MemType::DeviceAndPinned:
                gpuErrchk(fklhip_free(ref->ptr));
                gpuErrchk(fklhip_host_free(ref->pinnedPtr));
                break;
            }
            delete ref;
        }
        ref = nullptr;
    }

    void copyRaw(const RawPtr<D, T>& from, RawPtr<D, T>& to, int kind, void* stream) const {
        const bool tightFrom = from.dims.pitch == from.dims.width * sizeof(T);
        const bool tightTo = to.dims.pitch == to.dims.width * sizeof(T);
        if (tightFrom && tightTo) {
            if (L::bytes(from.dims) != L::bytes(to.dims)) throw std::runtime_error("Size mismatch in upload.");
            gpuErrchk(fklhip_memcpy_async(to.data, from.data, L::bytes(from.dims), kind, stream));
        } else {
            if constexpr (D != ND::_2D) {
                throw std::runtime_error("Padding only supported in 2D pointers");
            } else {
                gpuErrchk(fklhip_memcpy2d_async(to.data, to.dims.pitch, from.data, from.dims.pitch,
                                                from.dims.width * sizeof(T), from.dims.height, kind, stream));
            }
        }
    }

public:
    Ptr() {}

    Ptr(const Ptr& other)
        : ref(other.ref), ptr_a(other.ptr_a), ptr_pinned(other.ptr_pinned), type(other.type), deviceID(other.deviceID) {
        retain();
    }
    Ptr(Ptr&& other) noexcept
        : ref(other.ref), ptr_a(other.ptr_a), ptr_pinned(other.ptr_pinned), type(other.type), deviceID(other.deviceID) {
        other.ref = nullptr;
    }
    Ptr& operator=(const Ptr& other) {
        if (this != &other) {
            freePtr();
            ref = other.ref; ptr_a = other.ptr_a; ptr_pinned = other.ptr_pinned; type = other.type; deviceID = other.deviceID;
            retain();
        }
        return *this;
    }
    Ptr& operator=(Ptr&& other) noexcept(false) {
        if (this != &other) {
            freePtr();
            ref = other.ref; ptr_a = other.ptr_a; ptr_pinned = other.ptr_pinned; type = other.type; deviceID = other.deviceID;
            other.ref = nullptr;
        }
        return *this;
    }

    Ptr(const PtrDims<D>& dims, const MemType& type_ = defaultMemType, const int& deviceID_ = 0) { allocPtr(dims, type_, deviceID_); }

    // Views over memory somebody else owns: never freed here.
    Ptr(T* data_, const PtrDims<D>& dims, const MemType& type_, const int& deviceID_) {
        if (type_ == MemType::DeviceAndPinned)
            throw std::runtime_error("DeviceAndPinned type requires an additional argument for the pinned pointer.");
        ptr_a.data = data_; ptr_a.dims = dims; ptr_pinned = ptr_a; type = type_; deviceID = deviceID_;
    }
    Ptr(const RawPtr<D, T>& data_, const MemType& type_, const int& deviceID_) {
        if (type_ == MemType::DeviceAndPinned)
            throw std::runtime_error("DeviceAndPinned type requires an additional argument for the pinned pointer.");
        ptr_a = data_; ptr_pinned = ptr_a; type = type_; deviceID = deviceID_;
    }
    Ptr(T* data_, T* pinned_data, const PtrDims<D>& dims, const MemType& type_, const int& deviceID_) {
        ptr_a.data = data_; ptr_a.dims = dims; ptr_pinned.data = pinned_data; ptr_pinned.dims = dims;
        type = type_; deviceID = deviceID_;
    }
    Ptr(RefPtr* ref_, const RawPtr<D, T>& ptr_a_, const RawPtr<D, T>& ptr_pinned_, const MemType& type_, const int& devID)
        : ref(ref_), ptr_a(ptr_a_), ptr_pinned(ptr_pinned_), type(type_), deviceID(devID) {
        retain();
    }

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

    void allocPtr(const PtrDims<D>& dims_, const MemType& type_ = defaultMemType, const int& deviceID_ = 0) {
        if (ref) throw std::runtime_error("Reference pointer already exists. Use a different constructor.");
        ptr_a.dims = dims_;
        ptr_pinned.dims = dims_;
        type = type_;
        deviceID = deviceID_;
        ref = new RefPtr();
        try {
            switch (type) {
            case MemType::Device:
                ptr_detail::on_device(deviceID, [&] { L::device_alloc(ptr_a); });
                ptr_pinned = ptr_a;
                break;
            case MemType::Host:
                L::tight(ptr_a.dims);
                ptr_a.data = static_cast<T*>(std::malloc(L::bytes(ptr_a.dims)));
                if (!ptr_a.data && L::bytes(ptr_a.dims) != 0) throw std::bad_alloc();
                ptr_pinned = ptr_a;
                break;
            case MemType::HostPinned:
                L::tight(ptr_a.dims);
                ptr_detail::on_device(deviceID, [&] {
                    gpuErrchk(fklhip_host_alloc(reinterpret_cast<void**>(&ptr_a.data), L::bytes(ptr_a.dims)));
                });
                ptr_pinned = ptr_a;
                break;
            case MemType::DeviceAndPinned:
                ptr_detail::on_device(deviceID, [&] {
                    L::device_alloc(ptr_a);
                    L::tight(ptr_pinned.dims);   // the host mirror is always tightly packed
                    gpuErrchk(fklhip_host_alloc(reinterpret_cast<void**>(&ptr_pinned.data), L::bytes(ptr_pinned.dims)));
                });
                break;
            }
        } catch (...) {
            delete ref;
            ref = nullptr;
            throw;
        }
        ref->ptr = ptr_a.data;
        ref->pinnedPtr = ptr_pinned.data;
    }

    ~Ptr() { try { freePtr(); } catch (...) {} }

    RawPtr<D, T> ptr() const { return ptr_a; }
    RawPtr<D, T> ptrPinned() const { return ptr_pinned; }
    operator RawPtr<D, T>() const { return ptr_a; }

    // Sub-view sharing ownership with this pointer.
    Ptr<D, T> crop(const Point p, const PtrDims<D>& newDims) {
        const RawPtr<D, T> view{At::point(p, ptr_a), newDims};
        if (type == MemType::DeviceAndPinned) {
            const RawPtr<D, T> pinnedView{At::point(p, ptr_pinned), newDims};
            return Ptr<D, T>(ref, view, pinnedView, type, deviceID);
        }
        return Ptr<D, T>(ref, view, view, type, deviceID);
    }

    PtrDims<D> dims() const { return ptr_a.dims; }
    MemType getMemType() const { return type; }
    int getDeviceID() const { return deviceID; }
    size_t sizeInBytes() const { return L::bytes(ptr_a.dims); }
    uint getNumElements() const { return L::elements(ptr_a.dims); }
    int getRefCount() const { return ref ? ref->cnt.load() : 0; }

    void uploadTo(Ptr<D, T>& other, void* stream = nullptr) {
        if (type != MemType::Host && type != MemType::HostPinned)
            throw std::runtime_error("Upload can only copy from Host or HostPinned pointers.");
        if (other.type != MemType::Device && other.type != MemType::DeviceAndPinned)
            throw std::runtime_error("Upload can only copy to Device pointers");
        copyRaw(ptr_a, other.ptr_a, FKLHIP_COPY_H2D, stream);
    }
    void downloadTo(Ptr<D, T>& other, void* stream = nullptr) {
        if (type != MemType::Device && type != MemType::DeviceAndPinned)
            throw std::runtime_error("Download can only copy from Device pointers.");
        if (other.type != MemType::Host && other.type != MemType::HostPinned)
            throw std::runtime_error("Download can only copy to Host or HostPinned pointers.");
        copyRaw(ptr_a, other.ptr_a, FKLHIP_COPY_D2H, stream);
    }
    // Mirror <-> device transfers of a DeviceAndPinned pointer; no-ops for the other kinds.
    void upload(Stream_<ParArch::GPU_AMD>& stream) {
        if (type == MemType::DeviceAndPinned) copyRaw(ptr_pinned, ptr_a, FKLHIP_COPY_H2D, stream.getNativeStream());
    }
    void download(Stream_<ParArch::GPU_AMD>& stream) {
        if (type == MemType::DeviceAndPinned) copyRaw(ptr_a, ptr_pinned, FKLHIP_COPY_D2H, stream.getNativeStream());
    }
    void upload(Stream_<ParArch::CPU>&) {}
    void download(Stream_<ParArch::CPU>&) {}

    T at(const Point p) const {
        if (type == MemType::Device) throw std::runtime_error("Cannot access data in Device memory from host code");
        return *At::cr_point(p, ptr_pinned);
    }
    T& at(const Point p) {
        if (type == MemType::Device) throw std::runtime_error("Cannot access data in Device memory from host code");
        return *At::point(p, ptr_pinned);
    }
    T at(const int x) const { return at(Point{x, 0, 0}); }
    T& at(const int x) { return at(Point{x, 0, 0}); }
    template <ND DN = D> std::enable_if_t<(DN == ND::_2D || DN == ND::_3D), T> at(const int x, const int y) const { return at(Point{x, y, 0}); }
    template <ND DN = D> std::enable_if_t<(DN == ND::_2D || DN == ND::_3D), T&> at(const int x, const int y) { return at(Point{x, y, 0}); }
    template <ND DN = D> std::enable_if_t<(DN == ND::_3D), T> at(const int x, const int y, const int z) const { return at(Point{x, y, z}); }
    template <ND DN = D> std::enable_if_t<(DN == ND::_3D), T&> at(const int x, const int y, const int z) { return at(Point{x, y, z}); }

    template <ND DN = D> std::enable_if_t<(DN == ND::_3D), Ptr<ND::_2D, T>> getPlane(const uint& plane) {
        if (plane >= ptr_a.dims.planes) throw std::runtime_error("Plane index out of bounds");
        const PtrDims<ND::_2D> d(ptr_a.dims.width, ptr_a.dims.height, ptr_a.dims.pitch);
        const PtrDims<ND::_2D> dp(ptr_pinned.dims.width, ptr_pinned.dims.height, ptr_pinned.dims.pitch);
        const Point p{0, 0, int(plane)};
        return Ptr<ND::_2D, T>(ref, RawPtr<ND::_2D, T>{At::point(p, ptr_a), d}, RawPtr<ND::_2D, T>{At::point(p, ptr_pinned), dp}, type, deviceID);
    }
};

template <typename T> class Ptr1D : public Ptr<ND::_1D, T> {
public:
    Ptr1D() {}
    Ptr1D(const uint& num_elems, const uint& size_in_bytes = 0, const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::_1D, T>(PtrDims<ND::_1D>(num_elems, size_in_bytes), type_, deviceID_) {}
    Ptr1D(const Ptr<ND::_1D, T>& other) : Ptr<ND::_1D, T>(other) {}
    Ptr1D(T* data_, const PtrDims<ND::_1D>& dims_, const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::_1D, T>(data_, dims_, type_, deviceID_) {}
    Ptr1D<T> crop1D(const Point p, const PtrDims<ND::_1D>& newDims) { return Ptr<ND::_1D, T>::crop(p, newDims); }
};

template <typename T> class Ptr2D : public Ptr<ND::_2D, T> {
public:
    Ptr2D() {}
    Ptr2D(const Size& size, const uint& pitch_ = 0, const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::_2D, T>(PtrDims<ND::_2D>(size.width, size.height, pitch_), type_, deviceID_) {}
    Ptr2D(const uint& width_, const uint& height_, const uint& pitch_ = 0, const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::_2D, T>(PtrDims<ND::_2D>(width_, height_, pitch_), type_, deviceID_) {}
    Ptr2D(const Ptr<ND::_2D, T>& other) : Ptr<ND::_2D, T>(other) {}
    Ptr2D(T* data_, const uint& width_, const uint& height_, const uint& pitch_, const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::_2D, T>(data_, PtrDims<ND::_2D>(width_, height_, pitch_), type_, deviceID_) {}
    Ptr2D<T> crop2D(const Point p, const PtrDims<ND::_2D>& newDims) { return Ptr<ND::_2D, T>::crop(p, newDims); }
    void Alloc(const Size& size, const uint& pitch_ = 0, const MemType& type_ = defaultMemType, const int& deviceID_ = 0) {
        this->freePtr();
        this->allocPtr(PtrDims<ND::_2D>(size.width, size.height, pitch_), type_, deviceID_);
    }
};

template <typename T> class Ptr3D : public Ptr<ND::_3D, T> {
public:
    Ptr3D(const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1, const uint& pitch_ = 0,
          const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::_3D, T>(PtrDims<ND::_3D>(width_, height_, planes_, color_planes_, pitch_), type_, deviceID_) {}
    Ptr3D(const Ptr<ND::_3D, T>& other) : Ptr<ND::_3D, T>(other) {}
    Ptr3D(T* data_, const PtrDims<ND::_3D>& dims_, const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::_3D, T>(data_, dims_, type_, deviceID_) {}
    Ptr3D<T> crop3D(const Point p, const PtrDims<ND::_3D>& newDims) { return Ptr<ND::_3D, T>::crop(p, newDims); }
};

// A 3-D pointer with the colour planes outermost (every image's first channel plane, then every second one, ...).
template <typename T> class PtrT3D : public Ptr<ND::T3D, T> {
public:
    PtrT3D(const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1,
           const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::T3D, T>(PtrDims<ND::T3D>(width_, height_, planes_, color_planes_), type_, deviceID_) {}
    PtrT3D(const Ptr<ND::T3D, T>& other) : Ptr<ND::T3D, T>(other) {}
    PtrT3D(T* data_, const PtrDims<ND::T3D>& dims_, const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::T3D, T>(data_, dims_, type_, deviceID_) {}
    PtrT3D<T> crop3D(const Point p, const PtrDims<ND::T3D>& newDims) { return Ptr<ND::T3D, T>::crop(p, newDims); }
};

// Contiguous batch of planes: rows are always tightly packed (pitch = sizeof(T) * width).
template <typename T> class Tensor : public Ptr<ND::_3D, T> {
public:
    Tensor() {}
    Tensor(const Tensor<T>& other) : Ptr<ND::_3D, T>(other) {}
    Tensor& operator=(const Tensor<T>& other) { Ptr<ND::_3D, T>::operator=(other); return *this; }
    Tensor(const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1,
           const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::_3D, T>(PtrDims<ND::_3D>(width_, height_, planes_, color_planes_, uint(sizeof(T)) * width_), type_, deviceID_) {}
    Tensor(T* data, const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1,
           const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::_3D, T>(data, PtrDims<ND::_3D>(width_, height_, planes_, color_planes_, uint(sizeof(T)) * width_), type_, deviceID_) {}
    void allocTensor(const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1,
                     const MemType& type_ = defaultMemType, const int& deviceID_ = 0) {
        this->freePtr();
        this->allocPtr(PtrDims<ND::_3D>(width_, height_, planes_, color_planes_, uint(sizeof(T)) * width_), type_, deviceID_);
    }
};

// The same batch with the colour planes outermost (the layout TensorTSplit writes and TensorTPack reads).  A view over
// caller-owned memory gets the tight pitches the allocating constructor would have chosen.
template <typename T> class TensorT : public Ptr<ND::T3D, T> {
    static PtrDims<ND::T3D> tightDims(const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_) {
        PtrDims<ND::T3D> d(width_, height_, planes_, color_planes_);
        ptr_detail::Layout<ND::T3D, T>::tight(d);
        return d;
    }

public:
    TensorT() {}
    TensorT(const TensorT<T>& other) : Ptr<ND::T3D, T>(other) {}
    TensorT& operator=(const TensorT<T>& other) { Ptr<ND::T3D, T>::operator=(other); return *this; }
    TensorT(const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1,
            const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::T3D, T>(PtrDims<ND::T3D>(width_, height_, planes_, color_planes_), type_, deviceID_) {}
    TensorT(T* data, const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1,
            const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : Ptr<ND::T3D, T>(data, tightDims(width_, height_, planes_, color_planes_), type_, deviceID_) {}
    void allocTensor(const uint& width_, const uint& height_, const uint& planes_, const uint& color_planes_ = 1,
                     const MemType& type_ = defaultMemType, const int& deviceID_ = 0) {
        this->freePtr();
        this->allocPtr(PtrDims<ND::T3D>(width_, height_, planes_, color_planes_), type_, deviceID_);
    }
};

} // namespace fk
#endif
