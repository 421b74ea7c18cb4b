// ReadSet<T>: a read that yields one constant for every element of an active grid.
// Interface counterpart: FK/algorithms/basic_ops/set.h:29-80.
#ifndef FK_AMD_SET_H
#define FK_AMD_SET_H
#include <fused_kernel/core/data/ptr_nd.h>
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
namespace fk {
template <typename T> struct ReadSetParams {
    T value;
    ActiveThreads size;
};
template <typename T> struct ReadSet : ReadOperation<T, ReadSetParams<T>, T, TF::DISABLED, ReadSet<T>> {
    using Parent = ReadOperation<T, ReadSetParams<T>, T, TF::DISABLED, ReadSet<T>>;
    using typename Parent::OperationDataType;
    using typename Parent::InstantiableType;
    FK_STATIC_STRUCT(ReadSet, ReadSet)
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.size.x; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) { return opData.params.size.y; }
    static constexpr uint num_elems_z(const Point, const OperationDataType& opData) { return opData.params.size.z; }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) { return opData.params.size; }
    using Parent::build;
    static constexpr InstantiableType build(const T& value, const ActiveThreads& activeThreads) { return {{{value, activeThreads}}}; }
    template <ND D> static constexpr InstantiableType build(const T& value, const PtrDims<D>& dims) {
        static_assert(D == ND::_1D || D == ND::_2D || D == ND::_3D || D == ND::T3D, "Unsupported ND type for ReadSet build.");
        if constexpr (D == ND::_1D) return build(value, ActiveThreads(dims.width, 1, 1));
        else if constexpr (D == ND::_2D) return build(value, ActiveThreads(dims.width, dims.height, 1));
        else return build(value, ActiveThreads(dims.width, dims.height, dims.planes));
    }
};
namespace amd {
template <typename T> struct Lower<ReadSet<T>> {
    static constexpr bool available = true;
    using type = fkd::ReadSet<dev_t<T>>;
    static typename type::Params params(const OperationData<ReadSet<T>>& d) {
        return typename type::Params{to_dev(d.params.value), d.params.size.x, d.params.size.y, d.params.size.z};
    }
};
} // namespace amd
} // namespace fk
#endif
