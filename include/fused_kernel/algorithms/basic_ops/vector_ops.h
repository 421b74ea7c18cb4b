// VectorReorder<T, i0, i1, i2, i3>: out[c] = in[i_c].  Interface counterpart: FK/algorithms/basic_ops/vector_ops.h:43-56.
#ifndef FK_AMD_VECTOR_OPS_H
#define FK_AMD_VECTOR_OPS_H
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
namespace fk {
template <typename T, int... Idx> struct VectorReorder : UnaryOperation<T, T, VectorReorder<T, Idx...>> {
    using Parent = UnaryOperation<T, T, VectorReorder<T, Idx...>>;
    FK_STATIC_STRUCT(VectorReorder, VectorReorder)
    static_assert(validCUDAVec<T>, "Non valid vector type: VectorReorder");
    static_assert(cn<T> >= 2, "Minimum number of channels to reorder: 2");
    static_assert(sizeof...(Idx) == cn<T>, "Wrong number of indexes for the vector type");
};
namespace amd {
template <typename T, int I0, int I1> struct Lower<VectorReorder<T, I0, I1>> {
    static constexpr bool available = true;
    using type = fkd::Reorder<dev_t<T>, I0, I1, 2, 3>;
    static typename type::Params params(const OperationData<VectorReorder<T, I0, I1>>&) { return {}; }
};
template <typename T, int I0, int I1, int I2> struct Lower<VectorReorder<T, I0, I1, I2>> {
    static constexpr bool available = true;
    using type = fkd::Reorder<dev_t<T>, I0, I1, I2, 3>;
    static typename type::Params params(const OperationData<VectorReorder<T, I0, I1, I2>>&) { return {}; }
};
template <typename T, int I0, int I1, int I2, int I3> struct Lower<VectorReorder<T, I0, I1, I2, I3>> {
    static constexpr bool available = true;
    using type = fkd::Reorder<dev_t<T>, I0, I1, I2, I3>;
    static typename type::Params params(const OperationData<VectorReorder<T, I0, I1, I2, I3>>&) { return {}; }
};
} // namespace amd
} // namespace fk
#endif
