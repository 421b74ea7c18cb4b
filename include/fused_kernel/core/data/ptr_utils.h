// setTo(value, ptr, stream): fills every element of a Ptr with one value, as one fused launch
// (ReadSet -> PerThreadWrite).  Interface counterpart: FK/core/data/ptr_utils.h:24-45.
#ifndef FK_AMD_PTR_UTILS_H
#define FK_AMD_PTR_UTILS_H

#include <fused_kernel/algorithms/basic_ops/memory_operations.h>
#include <fused_kernel/algorithms/basic_ops/set.h>
#include <fused_kernel/core/data/ptr_nd.h>
#include <fused_kernel/core/execution_model/data_parallel_patterns.h>
#include <fused_kernel/core/execution_model/executors.h>

namespace fk {

// The device copy of the Ptr is filled on the stream.  A DeviceAndPinned Ptr also gets its pinned host mirror
// filled, on the host and right away (the reference does this with its CPU executor, which this backend does not
// have; a fill is plain data movement, not a computation of the fused path).
template <ParArch PA, ND D, typename T> inline void setTo(const T& value, Ptr<D, T>& outputPtr, Stream_<PA>& stream) {
    if constexpr (D == ND::T3D) {
        // Every colour plane is filled: the planes of a transposed tensor follow each other at plane_pitch, so the whole
        // of it is one batch of planes * color_planes planes.  (The reference's PerThreadWrite<T3D> addresses colour
        // plane 0 only and leaves the others as they were.)
        const auto t = outputPtr.ptr();
        const RawPtr<ND::_3D, T> all{t.data, PtrDims<ND::_3D>(t.dims.width, t.dims.height, t.dims.planes * t.dims.color_planes, 1, t.dims.pitch)};
        Executor<TransformDPP<PA>>::executeOperations(stream, ReadSet<T>::build(value, all.dims), PerThreadWrite<ND::_3D, T>::build(all));
    } else {
        Executor<TransformDPP<PA>>::executeOperations(stream, ReadSet<T>::build(value, outputPtr.dims()),
                                                      PerThreadWrite<D, T>::build(outputPtr.ptr()));
    }
    if (outputPtr.getMemType() == MemType::DeviceAndPinned) {
        const auto host = outputPtr.ptrPinned();
        const auto dims = host.dims;      // the mirror has its own (tight) pitch
        uint rows = 1u;
        if constexpr (D == ND::_2D) rows = dims.height;
        else if constexpr (D == ND::_3D || D == ND::T3D) rows = dims.height * dims.planes * dims.color_planes;
        for (uint y = 0; y < rows; ++y) {
            T* row = reinterpret_cast<T*>(reinterpret_cast<char*>(host.data) + size_t(y) * dims.pitch);
            for (uint x = 0; x < dims.width; ++x) row[x] = value;
        }
    }
}

} // namespace fk
#endif
