// POD views handed to kernels: PtrDims<D>, RawPtr<D,T>, and host-side address arithmetic PtrAccessor<D>.
// Interface counterpart: FK/core/data/rawptr.h:25-157 (types), :195-260 (accessors).
#ifndef FK_AMD_RAWPTR_H
#define FK_AMD_RAWPTR_H

#include <fused_kernel/core/utils/utils.h>
#include <fused_kernel/core/data/nd.h>
#include <fused_kernel/core/data/point.h>

namespace fk {

template <ND D> struct PtrDims;

template <> struct PtrDims<ND::_1D> {
    uint width{0};
    uint pitch{0};
    constexpr PtrDims() {}
    constexpr PtrDims(uint width_, uint pitch_ = 0) : width(width_), pitch(pitch_) {}
};

template <> struct PtrDims<ND::_2D> {
    uint width{0};
    uint height{0};
    uint pitch{0};
    constexpr PtrDims() {}
    constexpr PtrDims(uint width_, uint height_, uint pitch_ = 0) : width(width_), height(height_), pitch(pitch_) {}
};

// Batch of images: plane z begins plane_pitch * color_planes bytes after plane z - 1.
template <> struct PtrDims<ND::_3D> {
    uint width{0};
    uint height{0};
    uint planes{0};
    uint color_planes{0};
    uint pitch{0};
    uint plane_pitch{0};
    constexpr PtrDims() {}
    constexpr PtrDims(uint width_, uint height_, uint planes_, uint color_planes_ = 1, uint pitch_ = 0)
        : width(width_), height(height_), planes(planes_), color_planes(color_planes_), pitch(pitch_),
          plane_pitch(pitch_ * height_) {}
};

template <> struct PtrDims<ND::T3D> {
    uint width{0};
    uint height{0};
    uint planes{0};
    uint color_planes{0};
    uint pitch{0};
    uint plane_pitch{0};
    uint color_planes_pitch{0};
    constexpr PtrDims() {}
    constexpr PtrDims(uint width_, uint height_, uint planes_, uint color_planes_ = 1)
        : width(width_), height(height_), planes(planes_), color_planes(color_planes_) {}
};

template <ND D, typename T> struct RawPtr {
    T* data{nullptr};
    PtrDims<D> dims{};
    using type = T;
    enum { NDim = static_cast<int>(D) };
};

template <ND D> struct PtrAccessor;

template <> struct PtrAccessor<ND::_1D> {
    template <typename T, typename BiggerType = T>
    static const BiggerType* cr_point(const Point p, const RawPtr<ND::_1D, T>& ptr) { return (const BiggerType*)ptr.data + p.x; }
    template <typename T, typename BiggerType = T>
    static BiggerType* point(const Point p, const RawPtr<ND::_1D, T>& ptr) { return (BiggerType*)ptr.data + p.x; }
};

template <> struct PtrAccessor<ND::_2D> {
    template <typename T, typename BiggerType = T>
    static const BiggerType* cr_point(const Point p, const RawPtr<ND::_2D, T>& ptr) {
        return (const BiggerType*)((const char*)ptr.data + (size_t(p.y) * ptr.dims.pitch)) + p.x;
    }
    template <typename T, typename BiggerType = T>
    static BiggerType* point(const Point p, const RawPtr<ND::_2D, T>& ptr) {
        return (BiggerType*)((char*)ptr.data + (size_t(p.y) * ptr.dims.pitch)) + p.x;
    }
};

template <> struct PtrAccessor<ND::_3D> {
    template <typename T, typename BiggerType = T>
    static const BiggerType* cr_point(const Point p, const RawPtr<ND::_3D, T>& ptr) {
        return (const BiggerType*)((const char*)ptr.data + (size_t(ptr.dims.plane_pitch) * ptr.dims.color_planes * p.z) +
                                   (size_t(p.y) * ptr.dims.pitch)) + p.x;
    }
    template <typename T, typename BiggerType = T>
    static BiggerType* point(const Point p, const RawPtr<ND::_3D, T>& ptr) {
        return (BiggerType*)((char*)ptr.data + (size_t(ptr.dims.plane_pitch) * ptr.dims.color_planes * p.z) +
                             (size_t(p.y) * ptr.dims.pitch)) + p.x;
    }
};

// Channel planes outermost: channel plane c of image z starts c * color_planes_pitch + z * plane_pitch bytes in.
template <> struct PtrAccessor<ND::T3D> {
    template <typename T, typename BiggerType = T>
    static const BiggerType* cr_point(const Point p, const RawPtr<ND::T3D, T>& ptr, const uint color_plane = 0) {
        return (const BiggerType*)((const char*)ptr.data + (size_t(color_plane) * ptr.dims.color_planes_pitch) +
                                   (size_t(ptr.dims.plane_pitch) * p.z) + (size_t(p.y) * ptr.dims.pitch)) + p.x;
    }
    template <typename T, typename BiggerType = T>
    static BiggerType* point(const Point p, const RawPtr<ND::T3D, T>& ptr, const uint color_plane = 0) {
        return (BiggerType*)((char*)ptr.data + (size_t(color_plane) * ptr.dims.color_planes_pitch) +
                             (size_t(ptr.dims.plane_pitch) * p.z) + (size_t(p.y) * ptr.dims.pitch)) + p.x;
    }
};

// Small arrays with compile-time extents held by value (transform matrices and the like).
// Interface counterpart: FK/core/data/rawptr.h:105-185.
template <int W> struct StaticPtrDims1D { static constexpr uint width{W}; };
template <int W, int H> struct StaticPtrDims2D { static constexpr uint width{W}; static constexpr uint height{H}; };
template <int W, int H, int P> struct StaticPtrDims3D {
    static constexpr uint width{W}; static constexpr uint height{H}; static constexpr uint planes{P};
};
template <typename Dims, typename T> struct StaticRawPtr;
template <typename T, int W> struct StaticRawPtr<StaticPtrDims1D<W>, T> {
    using type = T;
    T data[W];
    static constexpr StaticPtrDims1D<W> dims{};
    static constexpr ND NDim{ND::_1D};
};
template <typename T, int W, int H> struct StaticRawPtr<StaticPtrDims2D<W, H>, T> {
    using type = T;
    T data[H][W];
    static constexpr StaticPtrDims2D<W, H> dims{};
    static constexpr ND NDim{ND::_2D};
};
template <typename T, int W, int H, int P> struct StaticRawPtr<StaticPtrDims3D<W, H, P>, T> {
    using type = T;
    T data[P][H][W];
    static constexpr StaticPtrDims3D<W, H, P> dims{};
    static constexpr ND NDim{ND::_3D};
};

} // namespace fk
#endif
